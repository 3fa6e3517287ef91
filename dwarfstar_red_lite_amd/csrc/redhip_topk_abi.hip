// C-ABI front end of the resident top-k expert pool (redmetal_topk_*): slots of raw GGUF expert bytes (gate|up|down) in
// HBM, filled by pread from the model file, and the weighted top-k FFN over a slot list - synchronous on host pointers, or
// enqueued on a HIP stream on device pointers, with the slot list given by the host or read from a device table. The
// arithmetic runs in the raw-format kernels of redhip_kernels.hip, which address an expert through a table of base addresses.
//
// Reference behaviour: native/redmetal_topk.m:1125-2062 (the pool object :700-1080); include/redmetal_topk.h cites each entry.
#include <fcntl.h>
#include <sys/stat.h>

#include <algorithm>
#include <mutex>
#include <vector>

#include "../../include/redmetal_topk.h"
#include "redhip_host_util.h"
#include "redhip_internal.h"

using namespace redhip;

namespace {

thread_local char g_topk_error[512];
#define TOPK_ERR(...) set_err(g_topk_error, sizeof(g_topk_error), __VA_ARGS__)

uint64_t round_up(uint64_t v, uint64_t a) { return v > UINT64_MAX - (a - 1u) ? 0u : (v + a - 1u) / a * a; }

struct TopkPool {
    int fd = -1;
    uint64_t file_size = 0, budget = 0, allocated = 0;
    uint32_t capacity = 0, slots_per_slab = 0;
    // slot size classes: slots cls_first[c] .. cls_first[c + 1) hold cls_bytes[c] each, their slabs are cls_slab[c] ..
    uint32_t n_cls = 1;
    uint32_t cls_first[RL_TOPK_MAX_CLASSES + 1] = {0}, cls_slab[RL_TOPK_MAX_CLASSES + 1] = {0};
    uint64_t cls_bytes[RL_TOPK_MAX_CLASSES] = {0};
    std::vector<uint8_t *> slab_of;               // by slab index over all classes; nullptr until first use
    uint32_t slabs_made = 0;
    std::vector<uint32_t> inflight, generation;
    std::mutex mu;                                // counters, slab creation, marks, residency mirror
    std::mutex exec_mu;                           // `execute` stages through buffers of the pool: one at a time
    std::recursive_mutex enc_mu;                  // an encode call sizes and fills buffers of the pool: host side one call at a time
    uint64_t bytes_read = 0, read_calls = 0;
    double read_ms = 0.0;
    std::vector<int8_t> iq2_xs, iq1_m;
    // buffers between the launches of a call (grow-only)
    DevBuf act, tmp, io;
    // the batched / mapped forms keep buffers of their own (the reference's _tmpB): growing them for a large chunk never moves `tmp`,
    // whose address callers hold through redmetal_topk_pool_tmp_buffer
    DevBuf act_b, tmp_b;
    // host lists of a call (slot addresses, weights, pair arrays) travel through a ring of pinned host buffers, each with a
    // device buffer of its own; an event recorded behind the call's last launch says when both may be used again
    struct Stage {
        void *host = nullptr, *host_dev = nullptr, *dev = nullptr;      // host_dev: the pinned buffer as the device addresses it
        size_t cap = 0;
        hipEvent_t done = nullptr;
        bool used = false;
    };
    static constexpr int kStages = 4;
    Stage stage[kStages];
    int next_stage = 0;
    // Opt-in fast path for one declared expert shape: behind the raw bytes of a slot lies a second copy in the layout the slice kernels
    // read (packed gate | up streams, column-sliced down), written when the slot is loaded. The copy of a slot starts shadow_off behind
    // the slot's address, the same distance in every slot, so a device-side slot table needs no second table.
    // kind 0: all IQ2_XXS; 1: IQ2_XXS gate / up with IQ3_S down (column-sliced words); 2 / 3: all IQ2_XS / all IQ1_M (streams decoded
    // through the pool's codebooks). gate / down: raw bytes of a matrix, gate_copy / down_copy: bytes of its re-laid form.
    // With REDHIP_TOPK_FAST_TILES a third copy follows tile_off behind the slot's address: the three matrices tile-major
    // (as large as the second copy), as the prefill tile kernels read them; the batched form then runs on those kernels.
    struct FastShape {
        uint32_t word = 0, hidden = 0, ffn = 0, kind = 0;
        uint64_t gate = 0, down = 0, gate_copy = 0, down_copy = 0, shadow_off = 0, tile_off = 0, slot_need = 0;
        bool tiles = false;
    };
    bool fast = false;
    FastShape fs;
    uint64_t cls_shadow[RL_TOPK_MAX_CLASSES] = {0};   // bytes behind each slot of the class for its copy (0: the class holds none)
    std::vector<uint8_t> shadow_ok;               // by slot: the copy matches the slot's raw bytes
    DevBuf partial;                               // partial output vectors of the slice kernels
    DevBuf stage_down;                            // load: the row-major packed down matrix on its way to the tile-major copy
    DevBuf chunk;                                 // batched form on the tile kernels: fp16 halves of x and of the activations, tile lists
    uint64_t phys(uint32_t c) const { return cls_bytes[c] + cls_shadow[c]; }
    uint32_t *iota = nullptr;                     // device [REDMETAL_TOPK_MAX + 1]: 0, 1, 2, .. (one pair per expert)
    uint64_t *residency = nullptr;                // device [layers][experts]
    uint32_t res_layers = 0, res_experts = 0;

    uint32_t class_of(uint32_t slot) const {
        uint32_t c = 0;
        while (c + 1u < n_cls && slot >= cls_first[c + 1u]) ++c;
        return c;
    }
    uint64_t bytes_for_slot(uint32_t slot) const { return slot < capacity ? cls_bytes[class_of(slot)] : 0u; }

    // device address of a slot; its slab is created on first use, within the budget. nullptr + message on failure
    uint8_t *slot_base(uint32_t slot) {
        if (slot >= capacity) { TOPK_ERR("top-k slot %u exceeds capacity %u", slot, capacity); return nullptr; }
        const uint32_t c = class_of(slot), in_class = slot - cls_first[c];
        const uint32_t slab = cls_slab[c] + in_class / slots_per_slab, local = in_class % slots_per_slab;
        std::lock_guard<std::mutex> lk(mu);
        if (!slab_of[slab]) {
            const uint32_t first = in_class / slots_per_slab * slots_per_slab, remaining = (cls_first[c + 1u] - cls_first[c]) - first;
            const uint64_t bytes = (uint64_t)(remaining < slots_per_slab ? remaining : slots_per_slab) * phys(c);
            if (!bytes || allocated > budget - bytes) { TOPK_ERR("top-k slab allocation would exceed hard budget"); return nullptr; }
            void *p = nullptr;
            const hipError_t e = hipMalloc(&p, (size_t)bytes);
            if (e != hipSuccess) { TOPK_ERR("failed to allocate top-k slab %.2f MiB: %s", (double)bytes / (1024.0 * 1024.0), hipGetErrorString(e)); return nullptr; }
            slab_of[slab] = static_cast<uint8_t *>(p);
            allocated += bytes;
            ++slabs_made;
        }
        return slab_of[slab] + (uint64_t)local * phys(c);
    }
    // may calls of this shape run on the slice kernels? (the copies of the slots they name are checked by the caller where it knows them)
    bool fast_shape(uint32_t word, uint32_t hidden, uint32_t ffn) const {
        return fast && hidden == fs.hidden && ffn == fs.ffn && word_gate_up(word) == word_gate_up(fs.word) && word_down(word) == word_down(fs.word);
    }
    void mark(const uint32_t *slots, uint32_t n, int delta) {
        std::lock_guard<std::mutex> lk(mu);
        for (uint32_t i = 0; i < n; ++i) {
            if (slots[i] >= capacity) continue;
            if (delta > 0) inflight[slots[i]] += 1u;
            else if (inflight[slots[i]]) inflight[slots[i]] -= 1u;
        }
    }
};

TopkPool *pool_of(redmetal_topk_pool_t h) { return static_cast<TopkPool *>(h); }

// What the raw-row kernels of this pool can stage in LDS: one token keeps its activation vector (hidden floats, padded) within the
// default 64 KB; the batched forms and the down rows keep eight pairs' vectors within 160 KB. Checked before anything is enqueued.
constexpr uint32_t kPoolMaxHiddenToken = 15360u, kPoolMaxBatched = 4864u;
bool pool_shape_ok(uint32_t hidden, uint32_t ffn, bool batched) {
    const uint32_t max_hidden = batched ? kPoolMaxBatched : kPoolMaxHiddenToken;
    if (hidden > max_hidden || ffn > kPoolMaxBatched) {
        TOPK_ERR("top-k shape hidden=%u ffn=%u exceeds what this pool's kernels stage in LDS (hidden <= %u, ffn <= %u for this call)", hidden, ffn, max_hidden, kPoolMaxBatched);
        return false;
    }
    return true;
}

bool type_word_ok(uint32_t w) { return !(w >> 16) && pool_quant_supported(word_gate_up(w)) && pool_quant_supported(word_down(w)); }

// this pool's codebooks on the device before an IQ2_XS / IQ1_M expert runs (free when they already are)
bool bind_grids(TopkPool *p, uint32_t type_word) {
    const uint32_t gu = word_gate_up(type_word), dn = word_down(type_word);
    if (gu != T_IQ2_XS && gu != T_IQ1_M && dn != T_IQ2_XS && dn != T_IQ1_M) return true;
    const hipError_t e = set_caller_grids(p->iq2_xs.data(), p->iq1_m.data(), p);
    if (e == hipErrorContextAlreadyInUse) { TOPK_ERR("%s", kCodebookConflict); return false; }
    if (e != hipSuccess) { TOPK_ERR("failed to upload the IQ2_XS / IQ1_M codebooks: %s", hipGetErrorString(e)); return false; }
    return true;
}

// native/redmetal_topk.m:1291-1336
bool validate(TopkPool *p, const uint32_t *slot_ids, const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes,
              uint32_t top_k, uint32_t type_word, uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count, bool batched = false) {
    if (!p || !slot_ids || !gate_bytes || !up_bytes || !down_bytes) return false;
    if (!top_k || top_k > REDMETAL_TOPK_MAX) { TOPK_ERR("top_k=%u must be in [1,%u]", top_k, REDMETAL_TOPK_MAX); return false; }
    if (!type_word_ok(type_word)) { TOPK_ERR("unsupported top-k GGML type word 0x%x (supported: IQ2_XS 17, IQ1_M 29, IQ2_XXS 16, IQ3_S 21, Q6_K 14)", type_word); return false; }
    if (!hidden || hidden % 256u || !ffn || ffn % 256u || !row_count || row_start >= hidden || row_count > hidden - row_start) {
        TOPK_ERR("invalid top-k dimensions hidden=%u ffn=%u start=%u count=%u", hidden, ffn, row_start, row_count);
        return false;
    }
    if (!pool_shape_ok(hidden, ffn, batched)) return false;
    if (top_k <= 32u) {
        for (uint32_t i = 0; i < top_k; ++i) {
            if (slot_ids[i] >= p->capacity) { TOPK_ERR("top-k slot %u exceeds capacity %u", slot_ids[i], p->capacity); return false; }
            for (uint32_t j = 0; j < i; ++j)
                if (slot_ids[i] == slot_ids[j]) { TOPK_ERR("top-k slot list contains duplicate slot %u", slot_ids[i]); return false; }
        }
    } else {                                            // long lists (the batched form): one pass over a sorted copy's neighbours
        std::vector<uint32_t> sorted(slot_ids, slot_ids + top_k);
        for (uint32_t v : sorted) if (v >= p->capacity) { TOPK_ERR("top-k slot %u exceeds capacity %u", v, p->capacity); return false; }
        std::sort(sorted.begin(), sorted.end());
        for (uint32_t i = 1; i < top_k; ++i)
            if (sorted[i] == sorted[i - 1u]) { TOPK_ERR("top-k slot list contains duplicate slot %u", sorted[i]); return false; }
    }
    const uint64_t expect_gate = (uint64_t)ffn * pool_row_bytes(word_gate_up(type_word), hidden);
    const uint64_t expect_down = (uint64_t)hidden * pool_row_bytes(word_down(type_word), ffn);
    for (uint32_t i = 0; i < top_k; ++i) {
        if (gate_bytes[i] != expect_gate || up_bytes[i] != expect_gate || down_bytes[i] != expect_down) { TOPK_ERR("top-k expert %u matrix byte mismatch", i); return false; }
        if (sizes_overflow(gate_bytes[i], up_bytes[i], down_bytes[i]) || gate_bytes[i] + up_bytes[i] + down_bytes[i] > p->bytes_for_slot(slot_ids[i])) {
            TOPK_ERR("top-k expert %u exceeds slot bounds", i);
            return false;
        }
    }
    return true;
}

bool ensure_scratch(TopkPool *p, uint32_t n_act_rows, uint32_t hidden, uint32_t ffn, bool batched = false) {
    DevBuf &act = batched ? p->act_b : p->act, &tmp = batched ? p->tmp_b : p->tmp;
    if (!act.reserve((size_t)n_act_rows * ffn * sizeof(float)) || !tmp.reserve((size_t)n_act_rows * hidden * sizeof(float))) {
        TOPK_ERR("failed to allocate top-k activation buffers");
        return false;
    }
    return true;
}

// the three launches of one token over a device slot table: gate/up + SwiGLU per expert, down rows per expert into tmp[e][r],
// weighted sum in list order (native/redmetal_topk.m:1338-1415 and :1858-1943). x1: experts from x_split on read it. With
// out == nullptr the sum is left to the caller; with a tail the last launch also adds the residual and the shared expert.
struct Tail { const float *resid, *shared, *scalar; float *x, *layer_out; };
constexpr uint32_t kFastMaxTopK = 64u;             // experts per call on the slice kernels (sizes the partial vectors)

__global__ __launch_bounds__(256) void topk_tail_kernel(const float *tmp, const float *weights, uint32_t top_k, uint32_t n,
                                                        const float *resid, const float *shared, const float *scalar, float *x, float *layer_out) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    float routed = 0.0f;
    for (uint32_t e = 0; e < top_k; ++e) routed = fmaf(weights[e], tmp[(uint64_t)e * n + i], routed);
    const float v = resid[i] + (routed + shared[i] * scalar[0]);
    x[i] = v;
    layer_out[i] = v;
}

bool enqueue_token(TopkPool *p, hipStream_t s, const uint64_t *table_dev, const float *weights_dev, uint32_t top_k, uint32_t type_word,
                   uint32_t hidden, uint32_t ffn, uint64_t gate_bytes, uint64_t up_bytes, uint32_t row_start, uint32_t row_count,
                   const float *x, const float *x1, uint32_t x_split, float *out, const Tail *tail, bool slots_fast) {
    std::lock_guard<std::recursive_mutex> lk(p->enc_mu);
    if (slots_fast && top_k <= kFastMaxTopK && row_start == 0u && row_count == hidden && (out || tail) && p->fast_shape(type_word, hidden, ffn)) {
        // two launches on the slots' re-laid copies: expert slices, then the sum of their partial vectors (with the tail when asked)
        float *partial = static_cast<float *>(p->partial.p);
        if (!bind_grids(p, type_word)) return false;
        const int8_t *grid = p->fs.kind >= 2u ? caller_grid_device(word_gate_up(type_word)) : nullptr;
        const hipError_t e = tail ? launch_slot_slices(table_dev, p->fs.shadow_off, weights_dev, top_k, hidden, ffn, x, x1, x_split, partial, tail->x,
                                                       tail->resid, tail->shared, tail->scalar, tail->layer_out, s, p->fs.kind, grid)
                                  : launch_slot_slices(table_dev, p->fs.shadow_off, weights_dev, top_k, hidden, ffn, x, x1, x_split, partial, out,
                                                       nullptr, nullptr, nullptr, nullptr, s, p->fs.kind, grid);
        if (e != hipSuccess) { TOPK_ERR("top-k HIP command failed: %s", hipGetErrorString(e)); return false; }
        return true;
    }
    if (!bind_grids(p, type_word) || !ensure_scratch(p, REDMETAL_TOPK_MAX, hidden, ffn)) return false;
    ExpertSet ex{nullptr, 0, gate_bytes, up_bytes, word_gate_up(type_word), word_down(type_word)};
    ex.table = table_dev;
    float *act = static_cast<float *>(p->act.p), *tmp = static_cast<float *>(p->tmp.p);
    hipError_t e = launch_moe_gateup(ex, nullptr, top_k, hidden, ffn, x, act, s, x1, x_split);
    // one group per expert with exactly one pair: pair e reads act[e], writes tmp[e]
    if (e == hipSuccess) e = launch_batch_down(ex, nullptr, p->iota, nullptr, top_k, top_k, hidden, ffn, act, tmp, s);
    if (e == hipSuccess && tail) {
        hipLaunchKernelGGL(topk_tail_kernel, dim3((hidden + 255u) / 256u), dim3(256), 0, s, tmp, weights_dev, top_k, hidden,
                           tail->resid, tail->shared, tail->scalar, tail->x, tail->layer_out);
        e = hipGetLastError();
    } else if (e == hipSuccess && out) {
        e = launch_weighted_sum(tmp, weights_dev, top_k, hidden, row_start, row_count, out, s);
    }
    if (e != hipSuccess) { TOPK_ERR("top-k HIP command failed: %s", hipGetErrorString(e)); return false; }
    return true;
}

__global__ __launch_bounds__(256) void stage_copy_kernel(uint4 *dst, const uint4 *src, uint32_t n16) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n16; i += gridDim.x * 256u) dst[i] = src[i];
}

// host lists of one call -> device through the next pinned stage. Layout: table u64 [n_table] | weights f32 [n_w] | u32 lists.
// The caller records the stage's event behind its last launch (stage_done).
struct Staged { uint64_t *table; float *w; uint32_t *u; TopkPool::Stage *stage; };
bool stage_lists(TopkPool *p, hipStream_t s, const std::vector<uint64_t> &table, const float *w, size_t n_w,
                 const std::vector<uint32_t> &u, Staged *out) {
    const size_t tb = table.size() * 8u, wb = (n_w * 4u + 7u) & ~(size_t)7u, ub = u.size() * 4u, total = tb + wb + ub;
    TopkPool::Stage *st;
    {
        std::lock_guard<std::mutex> lk(p->mu);
        st = &p->stage[p->next_stage];
        p->next_stage = (p->next_stage + 1) % TopkPool::kStages;
    }
    if (st->used && hipEventSynchronize(st->done) != hipSuccess) { TOPK_ERR("top-k staging buffer did not become free"); return false; }
    st->used = false;
    if (total > st->cap) {
        if (st->host) (void)hipHostFree(st->host);
        if (st->dev) (void)hipFree(st->dev);
        st->host = st->dev = nullptr;
        st->cap = 0;
        const size_t want = ((total < 65536u ? 65536u : total) + 15u) & ~(size_t)15u;
        if (hipHostMalloc(&st->host, want, hipHostMallocDefault) != hipSuccess || hipHostGetDevicePointer(&st->host_dev, st->host, 0) != hipSuccess ||
            hipMalloc(&st->dev, want) != hipSuccess ||
            (!st->done && hipEventCreateWithFlags(&st->done, hipEventDisableTiming) != hipSuccess)) {
            TOPK_ERR("failed to allocate top-k table buffers");
            return false;
        }
        st->cap = want;
    }
    uint8_t *host = static_cast<uint8_t *>(st->host), *base = static_cast<uint8_t *>(st->dev);
    memcpy(host, table.data(), tb);
    if (n_w) memcpy(host + tb, w, n_w * 4u);
    if (ub) memcpy(host + tb + wb, u.data(), ub);
    // a kernel reads the pinned buffer: the launches behind it follow in the same queue, without the hand-over between the copy engine
    // and the compute queue that a stream-ordered memcpy costs (tens of microseconds per call)
    const uint32_t n16 = (uint32_t)((total + 15u) / 16u);
    hipLaunchKernelGGL(stage_copy_kernel, dim3((n16 + 255u) / 256u < 64u ? (n16 + 255u) / 256u : 64u), dim3(256), 0, s, reinterpret_cast<uint4 *>(base),
                       static_cast<const uint4 *>(st->host_dev), n16);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) { TOPK_ERR("top-k table upload failed: %s", hipGetErrorString(e)); return false; }
    out->table = reinterpret_cast<uint64_t *>(base);
    out->w = reinterpret_cast<float *>(base + tb);
    out->u = reinterpret_cast<uint32_t *>(base + tb + wb);
    out->stage = st;
    return true;
}
void stage_done(const Staged &st, hipStream_t s) {
    if (hipEventRecord(st.stage->done, s) == hipSuccess) st.stage->used = true;
    else (void)hipStreamSynchronize(s);            // no event: the stage is free once the stream has drained
}

// batched experts over pairs sorted by expert: native/redmetal_topk.m:1474-1576. gate_table / down_table hold n_expert
// addresses each; up_delta is the distance from an expert's gate matrix to its up matrix, down_off the offset of the down
// matrix from its table entry.
bool enqueue_pairs(TopkPool *p, hipStream_t s, const std::vector<uint64_t> &gate_table, const std::vector<uint64_t> &down_table,
                   uint64_t up_delta, uint64_t down_off, uint32_t n_expert, uint32_t type_word, uint32_t hidden, uint32_t ffn,
                   uint32_t tok_first, uint32_t ntok, uint32_t top_k, uint32_t n_pairs, const uint32_t *pair_token,
                   const float *pair_weight, const uint32_t *expert_start, const uint32_t *tok_pair, const float *x, float *out) {
    std::lock_guard<std::recursive_mutex> lk(p->enc_mu);
    if (!bind_grids(p, type_word) || !ensure_scratch(p, n_pairs, hidden, ffn, true)) return false;
    std::vector<uint64_t> table(gate_table);
    table.insert(table.end(), down_table.begin(), down_table.end());
    std::vector<uint32_t> u;
    u.reserve((size_t)n_pairs * 2u + n_expert + 1u);
    u.insert(u.end(), pair_token, pair_token + n_pairs);
    u.insert(u.end(), expert_start, expert_start + n_expert + 1u);
    u.insert(u.end(), tok_pair, tok_pair + (size_t)ntok * top_k);
    Staged st;
    if (!stage_lists(p, s, table, pair_weight, n_pairs, u, &st)) return false;
    const uint32_t *d_pair_token = st.u, *d_start = st.u + n_pairs, *d_tok_pair = d_start + n_expert + 1u;
    float *act = static_cast<float *>(p->act_b.p), *tmp = static_cast<float *>(p->tmp_b.p);
    ExpertSet gu{nullptr, 0, up_delta, 0, word_gate_up(type_word), word_down(type_word)};
    gu.table = st.table;
    ExpertSet dn{nullptr, 0, down_off, 0, word_gate_up(type_word), word_down(type_word)};
    dn.table = st.table + n_expert;
    hipError_t e = launch_batch_gateup(gu, nullptr, d_start, d_pair_token, nullptr, n_expert, n_pairs, hidden, ffn, x, act, s);
    if (e == hipSuccess) e = launch_batch_down(dn, nullptr, d_start, nullptr, n_expert, n_pairs, hidden, ffn, act, tmp, s);
    if (e == hipSuccess) e = launch_batch_combine(tmp, st.w, d_tok_pair, ntok, top_k, nullptr, nullptr, hidden, out + (uint64_t)tok_first * hidden, s);
    stage_done(st, s);
    if (e != hipSuccess) { TOPK_ERR("batched top-k HIP command failed: %s", hipGetErrorString(e)); return false; }
    return true;
}

// The same pairs on the prefill tile kernels, for slots that hold tile-major copies: x split to fp16 halves per token, tiles of up to 32
// pairs per expert on the MFMA units (gate / up + SwiGLU, then down rows into tmp[pair]), combine in selection order. An expert is named
// by the distance of its slot from the lowest slot of the call, in units of 256 bytes (slots are 4096-aligned, HBM is far below 1 TB).
bool enqueue_pairs_tiles(TopkPool *p, hipStream_t s, const std::vector<uint64_t> &slot_addr, uint32_t n_expert, uint32_t hidden, uint32_t ffn,
                         uint32_t tok_first, uint32_t ntok, uint32_t top_k, uint32_t n_pairs, const uint32_t *pair_token, const float *pair_weight,
                         const uint32_t *expert_start, const uint32_t *tok_pair, const float *x, float *out) {
    std::lock_guard<std::recursive_mutex> lk(p->enc_mu);
    if (!bind_grids(p, p->fs.word)) return false;
    uint64_t lowest = slot_addr[0];
    for (uint64_t a : slot_addr) lowest = a < lowest ? a : lowest;
    std::vector<uint32_t> u;
    u.reserve((size_t)n_pairs * 2u + 2u * n_expert + 2u);
    u.insert(u.end(), pair_token, pair_token + n_pairs);
    u.insert(u.end(), expert_start, expert_start + n_expert + 1u);
    u.insert(u.end(), tok_pair, tok_pair + (size_t)ntok * top_k);
    for (uint64_t a : slot_addr) {
        const uint64_t d = a - lowest;
        if ((d & 255u) || (d >> 8) > 0xffffffffull) { TOPK_ERR("top-k slots of one call lie too far apart"); return false; }
        u.push_back((uint32_t)(d >> 8));
    }
    u.push_back(n_expert);
    // scratch of the call: rows of x up to the last token of the call, n_pairs activation rows
    const size_t rows = (size_t)tok_first + ntok, arows = (size_t)n_pairs + ntok;
    const uint32_t bound = prefill_tile_bound(ntok, top_k, n_expert);
    auto a256 = [](size_t v) { return (v + 255u) & ~(size_t)255u; };
    const size_t x_half = a256(rows * hidden * 2u), x_exp = a256(rows * 4u), a_half = a256(arows * ffn * 2u), a_exp = a256(arows * (ffn / 32u) * 4u), tl = a256(12u * (size_t)bound);
    if (!p->chunk.reserve(2u * x_half + 2u * x_exp + 2u * a_half + a_exp + 4u * tl) || !p->tmp_b.reserve((size_t)n_pairs * hidden * sizeof(float))) {
        TOPK_ERR("failed to allocate top-k activation buffers");
        return false;
    }
    uint8_t *w = static_cast<uint8_t *>(p->chunk.p);
    void *xh = w; w += x_half;
    void *xl = w; w += x_half;
    int *xexp = reinterpret_cast<int *>(w); w += x_exp;
    float *gate_unused = reinterpret_cast<float *>(w); w += x_exp;
    void *act_h = w; w += a_half;
    void *act_l = w; w += a_half;
    int *act_exp = reinterpret_cast<int *>(w); w += a_exp;
    uint32_t *tile_group = reinterpret_cast<uint32_t *>(w); w += tl;
    uint32_t *tile_pair0 = reinterpret_cast<uint32_t *>(w); w += tl;
    uint32_t *tile_n = reinterpret_cast<uint32_t *>(w); w += tl;
    uint32_t *n_tiles = reinterpret_cast<uint32_t *>(w);
    Staged st;
    if (!stage_lists(p, s, {}, pair_weight, n_pairs, u, &st)) return false;
    const uint32_t *d_pair_token = st.u, *d_start = st.u + n_pairs, *d_tok_pair = d_start + n_expert + 1u, *d_uid = d_tok_pair + (size_t)ntok * top_k, *d_unique = d_uid + n_expert;
    float *tmp = static_cast<float *>(p->tmp_b.p);
    const uint8_t *tiles = reinterpret_cast<const uint8_t *>(lowest + p->fs.tile_off);
    // (the split kernel also forms a gate logit per row from a second vector: x itself stands in, the result is not used)
    hipError_t e = launch_prep(x, x, (uint32_t)rows, hidden, xh, xl, xexp, gate_unused, s, nullptr, nullptr);
    if (e == hipSuccess && p->fs.kind == 0u)
        e = launch_prefill_packed(nullptr, 256u, nullptr, tiles, nullptr, d_uid, d_start, d_pair_token, d_unique, tile_group, tile_pair0, tile_n, n_tiles,
                                  xh, xl, xexp, act_h, act_l, act_exp, tmp, nullptr, hidden, ffn, top_k, ntok, n_expert, s, false, false);
    else if (e == hipSuccess && p->fs.kind == 1u) {      // IQ2_XXS gate / up tiles, then the IQ3_S down tiles
        e = launch_prefill_gateup_tiled(tiles, 256u, d_uid, d_start, d_pair_token, d_unique, tile_group, tile_pair0, tile_n, n_tiles, xh, xl, xexp, nullptr, act_h, act_l,
                                        act_exp, hidden, ffn, top_k, ntok, n_expert, s, false);
        if (e == hipSuccess)
            e = launch_prefill_down_iq3s(tiles + 2u * p->fs.gate_copy, 256u, d_uid, d_unique, tile_group, tile_pair0, tile_n, n_tiles, act_h, act_l, act_exp, tmp, hidden, ffn,
                                         top_k, ntok, n_expert, s);
    } else if (e == hipSuccess) {      // IQ2_XS / IQ1_M: the same tile kernels on the tile-major streams, through the pool's codebooks
        const uint32_t t = word_gate_up(p->fs.word);
        e = launch_prefill_streams(t, caller_grid_device(t), tiles, 256u, t, caller_grid_device(t), tiles + 2u * p->fs.gate_copy, 256u, d_uid, d_start, d_pair_token,
                                   d_unique, tile_group, tile_pair0, tile_n, n_tiles, xh, xl, xexp, act_h, act_l, act_exp, tmp, hidden, ffn, top_k, ntok, n_expert, s, false);
    }
    if (e == hipSuccess) e = launch_batch_combine(tmp, st.w, d_tok_pair, ntok, top_k, nullptr, nullptr, hidden, out + (uint64_t)tok_first * hidden, s);
    stage_done(st, s);
    if (e != hipSuccess) { TOPK_ERR("batched top-k HIP command failed: %s", hipGetErrorString(e)); return false; }
    return true;
}

bool pair_layout_ok(const char *what, uint32_t n_expert, uint32_t tok_first, uint32_t ntok, uint32_t top_k, uint32_t n_pairs,
                    const uint32_t *pair_token, const uint32_t *expert_start, const uint32_t *tok_pair) {
    if (expert_start[0] != 0u || expert_start[n_expert] != n_pairs) { TOPK_ERR("%s top-k expert_start is inconsistent", what); return false; }
    for (uint32_t u = 0; u < n_expert; ++u)
        if (expert_start[u] > expert_start[u + 1u]) { TOPK_ERR("%s top-k expert_start is inconsistent", what); return false; }
    for (uint32_t i = 0; i < n_pairs; ++i) if (pair_token[i] >= tok_first + ntok) { TOPK_ERR("%s top-k pair token out of range", what); return false; }
    for (uint32_t i = 0; i < ntok * top_k; ++i) if (tok_pair[i] >= n_pairs) { TOPK_ERR("%s top-k tok_pair out of range", what); return false; }
    return true;
}

float *at(void *dev, uint64_t byte_offset) { return reinterpret_cast<float *>(static_cast<uint8_t *>(dev) + byte_offset); }

int encode_device_impl(redmetal_topk_pool_t h, void *stream, void *slot_table_dev, uint64_t slot_table_offset, void *weight_dev,
                       uint64_t weight_offset, uint32_t top_k, uint32_t type_word, uint32_t hidden, uint32_t ffn, uint64_t gate_bytes,
                       uint64_t up_bytes, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset,
                       void *input1_dev, uint64_t input1_offset, uint32_t x_split, const Tail *tail) {
    TopkPool *p = pool_of(h);
    if (!p || !slot_table_dev || !weight_dev || !input_dev) return 0;
    if (!top_k || top_k > REDMETAL_TOPK_MAX || !type_word_ok(type_word) || !hidden || hidden % 256u || !ffn || ffn % 256u ||
        (slot_table_offset & 7u) || (weight_offset & 3u) || (input_offset & 15u)) {
        TOPK_ERR("invalid device-driven top-k request");
        return 0;
    }
    if (gate_bytes != (uint64_t)ffn * pool_row_bytes(word_gate_up(type_word), hidden) || up_bytes != gate_bytes) {
        TOPK_ERR("device-driven top-k matrix byte mismatch");
        return 0;
    }
    if (!pool_shape_ok(hidden, ffn, false)) return 0;
    const uint64_t *table = reinterpret_cast<const uint64_t *>(static_cast<uint8_t *>(slot_table_dev) + slot_table_offset);
    return enqueue_token(p, static_cast<hipStream_t>(stream), table, at(weight_dev, weight_offset), top_k, type_word, hidden, ffn,
                         gate_bytes, up_bytes, 0u, hidden, at(input_dev, input_offset), input1_dev ? at(input1_dev, input1_offset) : nullptr,
                         x_split, output_dev ? at(output_dev, output_offset) : nullptr, tail, true) ? 1 : 0;
}

}  // namespace

extern "C" {

uint32_t redmetal_topk_abi_version(void) { return 1u; }
const char *redmetal_topk_last_error(void) { return g_topk_error[0] ? g_topk_error : "unknown Red Metal top-k error"; }

redmetal_topk_pool_t redmetal_topk_pool_create(const char *model_path, uint64_t budget_bytes, uint64_t slot_bytes,
        uint32_t slots_per_slab, const int8_t *iq2_xs_grid, uint32_t iq2_xs_grid_count,
        const int8_t *iq1_m_grid, uint32_t iq1_m_grid_count) {
    g_topk_error[0] = '\0';
    if (!model_path || !model_path[0] || !budget_bytes || !slot_bytes || !iq2_xs_grid || !iq1_m_grid ||
        iq2_xs_grid_count != 512u * 8u || iq1_m_grid_count != 2048u * 8u) {
        TOPK_ERR("invalid Red Metal top-k pool arguments");
        return nullptr;
    }
    const uint64_t aligned = round_up(slot_bytes, 4096u);
    if (!aligned) { TOPK_ERR("top-k slot size overflow"); return nullptr; }
    if (aligned > budget_bytes) { TOPK_ERR("top-k cache budget cannot fit one aligned expert slot"); return nullptr; }
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { TOPK_ERR("no HIP device available"); return nullptr; }
    TopkPool *p = new TopkPool();
    p->iq2_xs.assign(iq2_xs_grid, iq2_xs_grid + iq2_xs_grid_count);
    p->iq1_m.assign(iq1_m_grid, iq1_m_grid + iq1_m_grid_count);
    p->budget = budget_bytes;
    const uint64_t cap64 = budget_bytes / aligned;
    p->capacity = cap64 > 0xffffffffull ? 0xffffffffu : (uint32_t)cap64;
    p->slots_per_slab = slots_per_slab ? slots_per_slab : 64u;
    if (p->slots_per_slab > p->capacity) p->slots_per_slab = p->capacity;
    p->n_cls = 1u;
    p->cls_bytes[0] = aligned;
    p->cls_first[0] = 0u;
    p->cls_first[1] = p->capacity;
    p->cls_slab[0] = 0u;
    p->cls_slab[1] = (p->capacity + p->slots_per_slab - 1u) / p->slots_per_slab;
    p->fd = open(model_path, O_RDONLY);
    if (p->fd < 0) { TOPK_ERR("open(%s) failed: %s", model_path, strerror(errno)); delete p; return nullptr; }
    struct stat st;
    if (fstat(p->fd, &st) != 0 || st.st_size <= 0) {
        TOPK_ERR("failed to stat model file: %s", strerror(errno));
        close(p->fd);
        delete p;
        return nullptr;
    }
    p->file_size = (uint64_t)st.st_size;
    p->inflight.assign(p->capacity, 0u);
    p->generation.assign(p->capacity, 0u);
    p->slab_of.assign(p->cls_slab[1], nullptr);
    std::vector<uint32_t> iota(REDMETAL_TOPK_MAX + 1u);
    for (uint32_t i = 0; i <= REDMETAL_TOPK_MAX; ++i) iota[i] = i;
    if (hipMalloc(reinterpret_cast<void **>(&p->iota), iota.size() * 4u) != hipSuccess ||
        hipMemcpy(p->iota, iota.data(), iota.size() * 4u, hipMemcpyHostToDevice) != hipSuccess) {
        TOPK_ERR("failed to allocate top-k table buffers");
        if (p->iota) (void)hipFree(p->iota);
        close(p->fd);
        delete p;
        return nullptr;
    }
    return p;
}

void redmetal_topk_pool_destroy(redmetal_topk_pool_t handle) {
    TopkPool *p = pool_of(handle);
    if (!p) return;
    (void)hipDeviceSynchronize();
    for (uint8_t *s : p->slab_of) if (s) (void)hipFree(s);
    if (p->iota) (void)hipFree(p->iota);
    if (p->residency) (void)hipFree(p->residency);
    for (TopkPool::Stage &st : p->stage) {
        if (st.host) (void)hipHostFree(st.host);
        if (st.dev) (void)hipFree(st.dev);
        if (st.done) (void)hipEventDestroy(st.done);
    }
    if (p->fd >= 0) close(p->fd);
    forget_caller_grids(p);
    delete p;
}

int redmetal_topk_pool_set_classes(redmetal_topk_pool_t handle, uint32_t n, const uint64_t *slot_bytes, const uint32_t *capacity) {
    TopkPool *p = pool_of(handle);
    if (!p) return 0;
    if (!n || n > RL_TOPK_MAX_CLASSES || !slot_bytes || !capacity) { TOPK_ERR("invalid top-k slot classes"); return 0; }
    std::lock_guard<std::mutex> lk(p->mu);
    if (p->slabs_made) { TOPK_ERR("top-k slot classes must be set before any slab is allocated"); return 0; }
    if (p->fast) { TOPK_ERR("top-k slot classes must be set before the fast path is enabled"); return 0; }
    uint64_t total = 0, sz[RL_TOPK_MAX_CLASSES];
    uint32_t slots = 0, slabs = 0, first[RL_TOPK_MAX_CLASSES + 1], slab[RL_TOPK_MAX_CLASSES + 1];
    for (uint32_t c = 0; c < n; ++c) {
        sz[c] = round_up(slot_bytes[c], 4096u);
        if (!sz[c] || !capacity[c] || (uint64_t)capacity[c] > UINT32_MAX - slots || sz[c] > (p->budget - total) / capacity[c]) {
            TOPK_ERR("top-k slot classes exceed the cache budget");
            return 0;
        }
        first[c] = slots;
        slab[c] = slabs;
        slots += capacity[c];
        total += sz[c] * capacity[c];
        slabs += (capacity[c] + p->slots_per_slab - 1u) / p->slots_per_slab;
    }
    first[n] = slots;
    slab[n] = slabs;
    p->n_cls = n;
    p->capacity = slots;
    for (uint32_t c = 0; c <= n; ++c) { p->cls_first[c] = first[c]; p->cls_slab[c] = slab[c]; }
    for (uint32_t c = 0; c < n; ++c) p->cls_bytes[c] = sz[c];
    p->inflight.assign(slots, 0u);
    p->generation.assign(slots, 0u);
    p->slab_of.assign(slabs, nullptr);
    return 1;
}

int redhip_topk_pool_enable_fast_path(redmetal_topk_pool_t handle, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint32_t flags) {
    TopkPool *p = pool_of(handle);
    if (!p) return 0;
    const uint32_t gu = type_word_ok(ggml_type) ? word_gate_up(ggml_type) : 0u, dn = type_word_ok(ggml_type) ? word_down(ggml_type) : 0u;
    const uint32_t kind = gu == T_IQ2_XXS && dn == T_IQ2_XXS ? 0u : gu == T_IQ2_XXS && dn == T_IQ3_S ? 1u : gu == T_IQ2_XS && dn == T_IQ2_XS ? 2u : gu == T_IQ1_M && dn == T_IQ1_M ? 3u : 4u;
    if (kind > 3u || !fused_iq2_supported(hidden_size, ffn_size) || hidden_size % 32u || (kind != 0u && hidden_size > 2048u)) {
        TOPK_ERR("the top-k fast path takes all-IQ2_XXS experts with hidden in {512, 1024, 2048, 4096}, or IQ2_XXS gate / up with IQ3_S down, all-IQ2_XS or all-IQ1_M experts with "
                 "hidden in {512, 1024, 2048}; ffn a multiple of 256 up to 1024 (asked: type word 0x%x, hidden=%u, ffn=%u)", ggml_type, hidden_size, ffn_size);
        return 0;
    }
    if ((flags & ~REDHIP_TOPK_FAST_TILES) || ((flags & REDHIP_TOPK_FAST_TILES) && (ffn_size > 512u || hidden_size > 2048u))) {
        TOPK_ERR("the top-k fast path keeps tile-major copies for hidden <= 2048 and ffn <= 512 only (asked: type word 0x%x, hidden=%u, ffn=%u, flags 0x%x)",
                 ggml_type, hidden_size, ffn_size, flags);
        return 0;
    }
    std::lock_guard<std::mutex> lk(p->mu);
    if (p->slabs_made) { TOPK_ERR("the top-k fast path must be enabled before any slab is allocated"); return 0; }
    if (p->fast) { TOPK_ERR("the top-k fast path is already enabled"); return 0; }
    TopkPool::FastShape f;
    f.word = ggml_type; f.hidden = hidden_size; f.ffn = ffn_size; f.kind = kind;
    f.gate = (uint64_t)ffn_size * pool_row_bytes(gu, hidden_size);
    f.down = (uint64_t)hidden_size * pool_row_bytes(dn, ffn_size);
    f.gate_copy = packed_matrix_bytes(gu, ffn_size, hidden_size);
    f.down_copy = kind == 1u ? iq3s_words_bytes(hidden_size, ffn_size) : packed_matrix_bytes(dn, hidden_size, ffn_size);
    const uint64_t payload = 2u * f.gate + f.down, copy_bytes = 2u * f.gate_copy + f.down_copy;
    f.tiles = (flags & REDHIP_TOPK_FAST_TILES) != 0u;
    f.shadow_off = round_up(payload, 256u);
    f.tile_off = f.shadow_off + round_up(copy_bytes, 256u);
    f.slot_need = round_up(f.tiles ? f.tile_off + copy_bytes : f.shadow_off + copy_bytes, 4096u);
    // classes that can hold an expert of this shape grow by the room for its copy; the budget covers both
    uint64_t shadow[RL_TOPK_MAX_CLASSES] = {0}, total = 0;
    bool any = false;
    for (uint32_t c = 0; c < p->n_cls; ++c) {
        if (p->cls_bytes[c] >= payload) {
            shadow[c] = f.slot_need > p->cls_bytes[c] ? f.slot_need - p->cls_bytes[c] : 0u;
            any = true;
        }
        total += (p->cls_bytes[c] + shadow[c]) * (uint64_t)(p->cls_first[c + 1u] - p->cls_first[c]);
    }
    if (!any) { TOPK_ERR("no top-k slot class holds an expert of the fast path's shape"); return 0; }
    if (p->n_cls == 1u) {
        // one class sized by the budget: fewer, larger slots
        const uint64_t cap64 = p->budget / (p->cls_bytes[0] + shadow[0]);
        if (!cap64) { TOPK_ERR("top-k cache budget cannot fit one expert slot with its copy"); return 0; }
        p->capacity = cap64 > 0xffffffffull ? 0xffffffffu : (uint32_t)cap64;
        if (p->slots_per_slab > p->capacity) p->slots_per_slab = p->capacity;
        p->cls_first[1] = p->capacity;
        p->cls_slab[1] = (p->capacity + p->slots_per_slab - 1u) / p->slots_per_slab;
        p->inflight.assign(p->capacity, 0u);
        p->generation.assign(p->capacity, 0u);
        p->slab_of.assign(p->cls_slab[1], nullptr);
    } else if (total > p->budget) {
        TOPK_ERR("top-k slot classes with the fast path's copies exceed the cache budget");
        return 0;
    }
    if (!p->partial.reserve((size_t)kFastMaxTopK * (ffn_size / 32u) * hidden_size * sizeof(float)) || (f.tiles && kind != 1u && !p->stage_down.reserve((size_t)f.down_copy))) {
        TOPK_ERR("failed to allocate top-k activation buffers");
        return 0;
    }
    for (uint32_t c = 0; c < p->n_cls; ++c) p->cls_shadow[c] = shadow[c];
    p->shadow_ok.assign(p->capacity, 0u);
    p->fs = f;
    p->fast = true;
    return 1;
}

uint32_t redmetal_topk_pool_capacity(redmetal_topk_pool_t h) { return h ? pool_of(h)->capacity : 0u; }
uint32_t redmetal_topk_pool_slab_count(redmetal_topk_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->slabs_made;
}
uint64_t redmetal_topk_pool_allocated_bytes(redmetal_topk_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->allocated;
}
uint64_t redmetal_topk_pool_bytes_read(redmetal_topk_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->bytes_read;
}
uint64_t redmetal_topk_pool_read_calls(redmetal_topk_pool_t h) {
    if (!h) return 0u;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->read_calls;
}
double redmetal_topk_pool_read_ms(redmetal_topk_pool_t h) {
    if (!h) return 0.0;
    std::lock_guard<std::mutex> lk(pool_of(h)->mu);
    return pool_of(h)->read_ms;
}
uint32_t redmetal_topk_pool_slot_generation(redmetal_topk_pool_t h, uint32_t slot_id) {
    TopkPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0u;
    std::lock_guard<std::mutex> lk(p->mu);
    return p->generation[slot_id];
}
int redmetal_topk_pool_slot_inflight(redmetal_topk_pool_t h, uint32_t slot_id) {
    TopkPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0;
    std::lock_guard<std::mutex> lk(p->mu);
    return p->inflight[slot_id] != 0u;
}

int redmetal_topk_pool_load_expert(redmetal_topk_pool_t h, uint32_t slot_id,
        uint64_t gate_file_offset, uint64_t gate_bytes, uint64_t up_file_offset, uint64_t up_bytes,
        uint64_t down_file_offset, uint64_t down_bytes, uint64_t *bytes_read, double *elapsed_ms) {
    TopkPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0;
    {
        std::lock_guard<std::mutex> lk(p->mu);
        if (p->inflight[slot_id]) { TOPK_ERR("refusing to overwrite in-flight top-k slot %u", slot_id); return 0; }
        p->generation[slot_id]++;
    }
    if (sizes_overflow(gate_bytes, up_bytes, down_bytes)) { TOPK_ERR("top-k expert payload size overflow"); return 0; }
    const uint64_t payload = gate_bytes + up_bytes + down_bytes;
    if (payload > p->bytes_for_slot(slot_id)) { TOPK_ERR("top-k expert payload exceeds slot size"); return 0; }
    uint8_t *base = p->slot_base(slot_id);
    if (!base) return 0;
    std::vector<uint8_t> host((size_t)payload);
    uint64_t local_bytes = 0, local_calls = 0;
    const double t0 = now_ms();
    const bool ok =
        pread_range(p->fd, p->file_size, gate_file_offset, gate_bytes, host.data(), &local_bytes, &local_calls, g_topk_error, sizeof(g_topk_error)) &&
        pread_range(p->fd, p->file_size, up_file_offset, up_bytes, host.data() + gate_bytes, &local_bytes, &local_calls, g_topk_error, sizeof(g_topk_error)) &&
        pread_range(p->fd, p->file_size, down_file_offset, down_bytes, host.data() + gate_bytes + up_bytes, &local_bytes, &local_calls, g_topk_error, sizeof(g_topk_error));
    if (!ok) return 0;
    if (payload) {
        const hipError_t e = hipMemcpy(base, host.data(), (size_t)payload, hipMemcpyHostToDevice);
        if (e != hipSuccess) { TOPK_ERR("top-k slot upload failed: %s", hipGetErrorString(e)); return 0; }
    }
    if (p->fast) {
        // the slot's copy for the slice kernels, when the expert has the declared shape and the slot's class has room for it
        const TopkPool::FastShape &f = p->fs;
        bool ok_copy = false;
        if (gate_bytes == f.gate && up_bytes == f.gate && down_bytes == f.down && f.slot_need <= p->phys(p->class_of(slot_id))) {
            uint8_t *copy = base + f.shadow_off, *tiles = base + f.tile_off;
            const uint32_t gu = word_gate_up(f.word), dn = word_down(f.word);
            hipError_t e = f.kind <= 1u ? launch_repack_iq2xxs(base, f.gate, 2u, f.ffn, f.hidden, false, copy, f.gate_copy, nullptr)
                                        : launch_repack_gateup(gu, base, f.gate, 2u, f.ffn, f.hidden, copy, f.gate_copy, nullptr);
            if (e == hipSuccess)
                e = f.kind == 0u   ? launch_repack_iq2xxs(base + 2u * f.gate, 0u, 1u, f.hidden, f.ffn, true, copy + 2u * f.gate_copy, 0u, nullptr)
                    : f.kind == 1u ? launch_repack_iq3s_words(base + 2u * f.gate, 0u, 1u, f.hidden, f.ffn, copy + 2u * f.gate_copy, 0u, nullptr, true)
                                   : launch_repack_gateup(dn, base + 2u * f.gate, 0u, 1u, f.hidden, f.ffn, copy + 2u * f.gate_copy, 0u, nullptr, true);
            if (f.tiles) {      // (kinds 0, 2, 3: the row-major packed down matrix passes through a staging buffer; IQ3_S tiles come from the raw rows)
                if (e == hipSuccess) e = launch_tile_packed(copy, f.gate_copy, 2u, f.ffn, f.hidden, tiles, f.gate_copy, nullptr, gu == T_IQ2_XS);
                if (e == hipSuccess && f.kind == 1u) e = launch_tile_iq3s(base + 2u * f.gate, 0u, 1u, f.hidden, f.ffn, tiles + 2u * f.gate_copy, 0u, nullptr);
                else if (e == hipSuccess)
                    e = f.kind == 0u ? launch_repack_iq2xxs(base + 2u * f.gate, 0u, 1u, f.hidden, f.ffn, false, p->stage_down.p, 0u, nullptr)
                                     : launch_repack_gateup(dn, base + 2u * f.gate, 0u, 1u, f.hidden, f.ffn, p->stage_down.p, 0u, nullptr);
                if (e == hipSuccess && f.kind != 1u) e = launch_tile_packed(p->stage_down.p, 0u, 1u, f.hidden, f.ffn, tiles + 2u * f.gate_copy, 0u, nullptr, dn == T_IQ2_XS);
            }
            if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
            if (e != hipSuccess) { TOPK_ERR("top-k slot re-layout failed: %s", hipGetErrorString(e)); return 0; }
            ok_copy = true;
        }
        std::lock_guard<std::mutex> lk(p->mu);
        p->shadow_ok[slot_id] = ok_copy ? 1u : 0u;
    }
    const double ms = now_ms() - t0;
    {
        std::lock_guard<std::mutex> lk(p->mu);
        p->bytes_read += local_bytes;
        p->read_calls += local_calls;
        p->read_ms += ms;
    }
    if (bytes_read) *bytes_read = local_bytes;
    if (elapsed_ms) *elapsed_ms = ms;
    return 1;
}

int redmetal_topk_pool_slot_addresses(redmetal_topk_pool_t h, uint32_t slot_id, uint64_t gate_bytes, uint64_t up_bytes,
        uint64_t down_bytes, uint64_t *gate_address, uint64_t *up_address, uint64_t *down_address) {
    TopkPool *p = pool_of(h);
    if (!p || slot_id >= p->capacity) return 0;
    if (sizes_overflow(gate_bytes, up_bytes, down_bytes) || gate_bytes + up_bytes + down_bytes > p->bytes_for_slot(slot_id)) return 0;
    uint8_t *base = p->slot_base(slot_id);
    if (!base) return 0;
    const uint64_t a = (uint64_t)(uintptr_t)base;
    if (gate_address) *gate_address = a;
    if (up_address) *up_address = a + gate_bytes;
    if (down_address) *down_address = a + gate_bytes + up_bytes;
    return 1;
}

int redmetal_topk_pool_encode(redmetal_topk_pool_t h, void *stream, const uint32_t *slot_ids,
        const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes,
        const float *router_weights, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
        uint32_t output_row_start, uint32_t output_row_count, void *input_dev, uint64_t input_offset,
        void *output_dev, uint64_t output_offset) {
    TopkPool *p = pool_of(h);
    if (!p || !router_weights || !input_dev || !output_dev) return 0;
    if (!validate(p, slot_ids, gate_bytes, up_bytes, down_bytes, top_k, ggml_type, hidden_size, ffn_size, output_row_start, output_row_count)) return 0;
    if ((input_offset & 15u) || (output_offset & 3u)) { TOPK_ERR("top-k external buffer offsets must keep the input 16-byte aligned"); return 0; }
    std::vector<uint64_t> table(top_k);
    for (uint32_t i = 0; i < top_k; ++i) {
        uint8_t *base = p->slot_base(slot_ids[i]);
        if (!base) return 0;
        table[i] = (uint64_t)(uintptr_t)base;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::recursive_mutex> lk(p->enc_mu);
    bool copies = p->fast;
    if (copies) {
        std::lock_guard<std::mutex> lk2(p->mu);
        for (uint32_t i = 0; i < top_k; ++i) copies = copies && p->shadow_ok[slot_ids[i]];
    }
    Staged st;
    if (!stage_lists(p, s, table, router_weights, top_k, {}, &st)) return 0;
    const bool ok = enqueue_token(p, s, st.table, st.w, top_k, ggml_type, hidden_size, ffn_size, gate_bytes[0], up_bytes[0], output_row_start,
                                  output_row_count, at(input_dev, input_offset), nullptr, 0u, at(output_dev, output_offset), nullptr, copies);
    stage_done(st, s);
    if (!ok) return 0;
    p->mark(slot_ids, top_k, +1);
    return 1;
}

void redmetal_topk_pool_release(redmetal_topk_pool_t h, const uint32_t *slot_ids, uint32_t top_k) {
    TopkPool *p = pool_of(h);
    if (!p || !slot_ids) return;
    p->mark(slot_ids, top_k, -1);
}

int redmetal_topk_pool_execute(redmetal_topk_pool_t h, const uint32_t *slot_ids,
        const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes,
        const float *router_weights, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
        uint32_t output_row_start, uint32_t output_row_count, const float *input, uint32_t input_count,
        float *output, uint32_t output_count, double *elapsed_ms) {
    TopkPool *p = pool_of(h);
    if (!p || !router_weights || !input || !output) return 0;
    if (!validate(p, slot_ids, gate_bytes, up_bytes, down_bytes, top_k, ggml_type, hidden_size, ffn_size, output_row_start, output_row_count)) return 0;
    if (input_count != hidden_size || output_count < output_row_count) { TOPK_ERR("invalid top-k host buffer sizes"); return 0; }
    std::lock_guard<std::mutex> exec(p->exec_mu);
    if (!p->io.reserve(2u * (size_t)hidden_size * sizeof(float))) { TOPK_ERR("failed to allocate top-k activation buffers"); return 0; }
    float *dx = static_cast<float *>(p->io.p), *dout = dx + hidden_size;
    hipError_t e = hipMemcpy(dx, input, (size_t)hidden_size * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) { TOPK_ERR("top-k input upload failed: %s", hipGetErrorString(e)); return 0; }
    const double t0 = now_ms();
    if (!redmetal_topk_pool_encode(h, nullptr, slot_ids, gate_bytes, up_bytes, down_bytes, router_weights, top_k, ggml_type, hidden_size, ffn_size,
                                   output_row_start, output_row_count, dx, 0u, dout, 0u)) return 0;
    e = hipStreamSynchronize(nullptr);
    const double ms = now_ms() - t0;
    p->mark(slot_ids, top_k, -1);
    if (e != hipSuccess) { TOPK_ERR("top-k HIP command failed: %s", hipGetErrorString(e)); return 0; }
    e = hipMemcpy(output, dout, (size_t)output_row_count * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) { TOPK_ERR("top-k output download failed: %s", hipGetErrorString(e)); return 0; }
    if (elapsed_ms) *elapsed_ms = ms;
    return 1;
}

int redmetal_topk_pool_residency_table_init(redmetal_topk_pool_t h, uint32_t layers, uint32_t experts) {
    TopkPool *p = pool_of(h);
    if (!p || !layers || !experts) return 0;
    const size_t bytes = (size_t)layers * experts * sizeof(uint64_t);
    std::lock_guard<std::mutex> lk(p->mu);
    if (p->residency) { (void)hipDeviceSynchronize(); (void)hipFree(p->residency); p->residency = nullptr; }
    if (hipMalloc(reinterpret_cast<void **>(&p->residency), bytes) != hipSuccess || hipMemset(p->residency, 0, bytes) != hipSuccess) {
        TOPK_ERR("failed to allocate the expert residency table");
        if (p->residency) { (void)hipFree(p->residency); p->residency = nullptr; }
        return 0;
    }
    p->res_layers = layers;
    p->res_experts = experts;
    return 1;
}

void *redmetal_topk_pool_residency_table(redmetal_topk_pool_t h) { return h ? pool_of(h)->residency : nullptr; }

int redmetal_topk_pool_residency_set(redmetal_topk_pool_t h, uint32_t layer, uint32_t expert, uint32_t slot_id) {
    TopkPool *p = pool_of(h);
    if (!p || !p->residency || layer >= p->res_layers || expert >= p->res_experts) return 0;
    uint8_t *base = p->slot_base(slot_id);
    if (!base) return 0;
    const uint64_t v = (uint64_t)(uintptr_t)base;
    return hipMemcpy(p->residency + (size_t)layer * p->res_experts + expert, &v, sizeof(v), hipMemcpyHostToDevice) == hipSuccess ? 1 : 0;
}

void redmetal_topk_pool_residency_clear(redmetal_topk_pool_t h, uint32_t layer, uint32_t expert) {
    TopkPool *p = pool_of(h);
    if (!p || !p->residency || layer >= p->res_layers || expert >= p->res_experts) return;
    const uint64_t v = 0u;
    (void)hipMemcpy(p->residency + (size_t)layer * p->res_experts + expert, &v, sizeof(v), hipMemcpyHostToDevice);
}

void *redmetal_topk_pool_slab_residency_set(redmetal_topk_pool_t) { return nullptr; }
void redmetal_topk_pool_use_all_slabs(redmetal_topk_pool_t, void *) {}

int redmetal_topk_pool_allocate_all(redmetal_topk_pool_t h) {
    TopkPool *p = pool_of(h);
    if (!p) return 0;
    for (uint32_t c = 0; c < p->n_cls; ++c)
        for (uint32_t s = p->cls_first[c]; s < p->cls_first[c + 1u]; s += p->slots_per_slab)
            if (!p->slot_base(s)) return 0;
    return 1;
}

void *redmetal_topk_pool_tmp_buffer(redmetal_topk_pool_t h) { return h ? pool_of(h)->tmp.p : nullptr; }

int redmetal_topk_pool_encode_device(redmetal_topk_pool_t h, void *stream, void *slot_table_dev, uint64_t slot_table_offset,
        void *weight_dev, uint64_t weight_offset, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
        uint64_t gate_bytes, uint64_t up_bytes, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset) {
    if (!output_dev) { TOPK_ERR("invalid device-driven top-k request"); return 0; }
    return encode_device_impl(h, stream, slot_table_dev, slot_table_offset, weight_dev, weight_offset, top_k, ggml_type, hidden_size, ffn_size,
                              gate_bytes, up_bytes, input_dev, input_offset, output_dev, output_offset, nullptr, 0u, 0u, nullptr);
}

int redmetal_topk_pool_encode_device_into(redmetal_topk_pool_t h, void *stream, void *slot_table_dev, uint64_t slot_table_offset,
        void *weight_dev, uint64_t weight_offset, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
        uint64_t gate_bytes, uint64_t up_bytes, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset) {
    return encode_device_impl(h, stream, slot_table_dev, slot_table_offset, weight_dev, weight_offset, top_k, ggml_type, hidden_size, ffn_size,
                              gate_bytes, up_bytes, input_dev, input_offset, output_dev, output_offset, nullptr, 0u, 0u, nullptr);
}

int redmetal_topk_pool_encode_device_into2(redmetal_topk_pool_t h, void *stream, void *slot_table_dev, uint64_t slot_table_offset,
        void *weight_dev, uint64_t weight_offset, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
        uint64_t gate_bytes, uint64_t up_bytes, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset,
        void *input1_dev, uint64_t input1_offset, uint32_t x_split) {
    if (input1_dev && (input1_offset & 15u)) { TOPK_ERR("invalid device-driven top-k request"); return 0; }
    return encode_device_impl(h, stream, slot_table_dev, slot_table_offset, weight_dev, weight_offset, top_k, ggml_type, hidden_size, ffn_size,
                              gate_bytes, up_bytes, input_dev, input_offset, output_dev, output_offset, input1_dev, input1_offset, x_split, nullptr);
}

int redmetal_topk_pool_encode_device_tail(redmetal_topk_pool_t h, void *stream, void *slot_table_dev, uint64_t slot_table_offset,
        void *weight_dev, uint64_t weight_offset, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
        uint64_t gate_bytes, uint64_t up_bytes, void *input_dev, uint64_t input_offset, void *resid_dev, void *shared_dev,
        void *scalar_dev, void *x_dev, void *layer_out_dev, uint64_t layer_out_offset) {
    if (!h || top_k > 64u) return -1;
    if (!resid_dev || !shared_dev || !scalar_dev || !x_dev || !layer_out_dev) { TOPK_ERR("invalid device-driven top-k request"); return 0; }
    const Tail tail{static_cast<const float *>(resid_dev), static_cast<const float *>(shared_dev), static_cast<const float *>(scalar_dev),
                    static_cast<float *>(x_dev), at(layer_out_dev, layer_out_offset)};
    return encode_device_impl(h, stream, slot_table_dev, slot_table_offset, weight_dev, weight_offset, top_k, ggml_type, hidden_size, ffn_size,
                              gate_bytes, up_bytes, input_dev, input_offset, nullptr, 0u, nullptr, 0u, 0u, &tail);
}

int redmetal_topk_pool_encode_batched(redmetal_topk_pool_t h, void *stream, const uint32_t *slot_ids,
        const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes, uint32_t n_expert,
        uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint32_t tok_first, uint32_t ntok, uint32_t top_k,
        uint32_t n_pairs, const uint32_t *pair_token, const float *pair_weight, const uint32_t *expert_start,
        const uint32_t *tok_pair, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset) {
    TopkPool *p = pool_of(h);
    if (!p || !input_dev || !output_dev || !pair_token || !pair_weight || !expert_start || !tok_pair) return 0;
    if (!ntok || !top_k || !n_pairs || (uint64_t)ntok * top_k != n_pairs || n_pairs > REDMETAL_TOPK_MAX * 64u) { TOPK_ERR("invalid batched top-k pair layout"); return 0; }
    if (!validate(p, slot_ids, gate_bytes, up_bytes, down_bytes, n_expert, ggml_type, hidden_size, ffn_size, 0u, hidden_size, true)) return 0;
    if (!pair_layout_ok("batched", n_expert, tok_first, ntok, top_k, n_pairs, pair_token, expert_start, tok_pair)) return 0;
    std::vector<uint64_t> table(n_expert);
    for (uint32_t i = 0; i < n_expert; ++i) {
        uint8_t *base = p->slot_base(slot_ids[i]);
        if (!base) return 0;
        table[i] = (uint64_t)(uintptr_t)base;
    }
    bool tiles = p->fast && p->fs.tiles && p->fast_shape(ggml_type, hidden_size, ffn_size) && n_expert <= 1024u;
    if (tiles) {
        std::lock_guard<std::mutex> lk(p->mu);
        for (uint32_t i = 0; i < n_expert; ++i) tiles = tiles && p->shadow_ok[slot_ids[i]];
    }
    if (tiles ? !enqueue_pairs_tiles(p, static_cast<hipStream_t>(stream), table, n_expert, hidden_size, ffn_size, tok_first, ntok, top_k, n_pairs, pair_token,
                                     pair_weight, expert_start, tok_pair, at(input_dev, input_offset), at(output_dev, output_offset))
              : !enqueue_pairs(p, static_cast<hipStream_t>(stream), table, table, gate_bytes[0], gate_bytes[0] + up_bytes[0], n_expert, ggml_type,
                               hidden_size, ffn_size, tok_first, ntok, top_k, n_pairs, pair_token, pair_weight, expert_start, tok_pair,
                               at(input_dev, input_offset), at(output_dev, output_offset))) return 0;
    p->mark(slot_ids, n_expert, +1);
    return 1;
}

int redmetal_topk_pool_encode_mapped(redmetal_topk_pool_t h, void *stream,
        void *, uint64_t gate_addr0, void *, uint64_t up_addr0, void *, uint64_t down_addr0,
        uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes, const uint32_t *expert_ids, uint32_t n_expert,
        uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint32_t tok_first, uint32_t ntok, uint32_t top_k,
        uint32_t n_pairs, const uint32_t *pair_token, const float *pair_weight, const uint32_t *expert_start,
        const uint32_t *tok_pair, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset) {
    TopkPool *p = pool_of(h);
    if (!p || !gate_addr0 || !up_addr0 || !down_addr0 || !expert_ids || !pair_token || !pair_weight || !expert_start || !tok_pair || !input_dev || !output_dev) return 0;
    if (!n_expert || n_expert > REDMETAL_TOPK_MAX || !ntok || !top_k || (uint64_t)ntok * top_k != n_pairs) { TOPK_ERR("invalid mapped top-k request"); return 0; }
    if (!type_word_ok(ggml_type) || !hidden_size || hidden_size % 256u || !ffn_size || ffn_size % 256u) { TOPK_ERR("mapped top-k needs a supported type word and 256-aligned sizes"); return 0; }
    if (gate_bytes != (uint64_t)ffn_size * pool_row_bytes(word_gate_up(ggml_type), hidden_size) || up_bytes != gate_bytes ||
        down_bytes != (uint64_t)hidden_size * pool_row_bytes(word_down(ggml_type), ffn_size)) { TOPK_ERR("mapped top-k matrix byte mismatch"); return 0; }
    if (!pool_shape_ok(hidden_size, ffn_size, true)) return 0;
    if (!pair_layout_ok("mapped", n_expert, tok_first, ntok, top_k, n_pairs, pair_token, expert_start, tok_pair)) return 0;
    std::vector<uint64_t> gate(n_expert), down(n_expert);
    for (uint32_t i = 0; i < n_expert; ++i) {
        gate[i] = gate_addr0 + (uint64_t)expert_ids[i] * gate_bytes;
        down[i] = down_addr0 + (uint64_t)expert_ids[i] * down_bytes;
    }
    // gate and up matrices have the same size, so the up matrix of every expert lies at the same distance from its gate matrix
    return enqueue_pairs(p, static_cast<hipStream_t>(stream), gate, down, up_addr0 - gate_addr0, 0u, n_expert, ggml_type, hidden_size, ffn_size,
                         tok_first, ntok, top_k, n_pairs, pair_token, pair_weight, expert_start, tok_pair,
                         at(input_dev, input_offset), at(output_dev, output_offset)) ? 1 : 0;
}

}  // extern "C"
