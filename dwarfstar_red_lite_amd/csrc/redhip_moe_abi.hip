// Resident MoE FFN layers: every expert of every layer stays in HBM, one call runs a layer's FFN on a stream.
// See include/redhip_moe.h for the contract.
#include <stdarg.h>
#include <stdlib.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "../../include/redhip_moe.h"
#include "redhip_internal.h"

using namespace redhip;

namespace {

thread_local char g_moe_error[512];
void moe_err(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_moe_error, sizeof(g_moe_error), fmt, ap);
    va_end(ap);
}
#define HIP_OK(call, what)                                                            \
    do {                                                                              \
        const hipError_t e_ = (call);                                                 \
        if (e_ != hipSuccess) { moe_err("%s: %s", what, hipGetErrorString(e_)); return 0; } \
    } while (0)

struct Layer {
    uint8_t *router = nullptr;       // [n_expert] rows of `hidden` weights (F32 or Q6_K)
    uint8_t *shared = nullptr;       // gate | up | down of the shared expert
    float *gate_inp = nullptr;       // [hidden]
    uint8_t *experts = nullptr;      // n_expert slots of expert_stride bytes, each gate | up | down
    uint8_t *packed = nullptr;       // same slots in the packed IQ2_XXS layout of the fused kernel (fused path only)
    uint8_t *shared_packed = nullptr;
    uint8_t *down_cm = nullptr;      // all-IQ2_XXS layers: the packed down matrices once more, column-sliced (qs [ffn / 32][hidden], ds [ffn / 256][hidden]), for the
    uint8_t *shared_down_cm = nullptr;      // slice kernels whose workgroups each take 32 columns of a down matrix; mixed layouts with IQ3_S down matrices
                                            // whose small batches run as slices: their word-packed down matrices column-sliced (no shared_down_cm)
    uint8_t *tiled = nullptr;        // third copy, tile-major, read by the prefill kernels (handles that take chunks only)
    uint8_t *shared_tiled = nullptr;
    // mixed layouts that take chunks: f32 copies of the small dense matrices (dequantised once at upload) for the fp32 tile
    // kernel: router [n_expert][hidden] (when it is quantised), shared gate | up [2 ffn][hidden], shared down [hidden][ffn]
    float *dense_router = nullptr, *dense_gu = nullptr, *dense_down = nullptr;
    uint8_t *tiled_down = nullptr;   // mixed layouts with IQ3_S, IQ2_XS or IQ1_M down matrices that take chunks on tile kernels: their tile-major copy
    uint8_t *words_down = nullptr;   // mixed layouts with IQ3_S / IQ2_XS / IQ1_M down matrices, row-major words or streams for the MFMA down kernels of up to 8 tokens (layers with a column-sliced IQ3_S copy read that one instead)
};

struct Moe {
    redhip_moe_config cfg;
    uint32_t gu_type, dn_type, sh_gu_type, sh_dn_type;
    uint64_t gate_bytes, down_bytes, expert_stride;          // routed expert
    uint64_t down_cm_stride() const { return mixed ? words_down_stride() : (down_bytes + 255u) & ~255ull; }
    float *partial = nullptr;                                // [tokens <= 8][top_k + 1][ffn / 32][hidden]: partial output vectors of the expert slices
    uint2 *pass_list = nullptr;                              // small batches: the passes (two pairs of one expert) of the batched expert slices
    uint32_t *n_pass = nullptr;
    uint64_t pk_gate_bytes = 0;                              // one gate / up matrix in the packed streams of the one-token kernel
    const int8_t *gu_grid = nullptr, *dn_grid = nullptr;     // device copies of the caller's codebooks (IQ2_XS / IQ1_M matrices)
    uint64_t sh_gate_bytes, sh_down_bytes;                   // shared expert
    uint64_t router_bytes;
    uint64_t resident = 0;
    std::vector<Layer> layers;
    // workspace (device), sized for max_tokens
    float *logits = nullptr, *weights = nullptr, *scalar = nullptr, *act = nullptr, *sh_act = nullptr;
    float *xn = nullptr;                     // [max_tokens][hidden]: normalised activations of redhip_moe_forward_block
    uint32_t *ids = nullptr;
    uint32_t *status = nullptr;              // device word: bit 0 an expert id of the caller's routing was out of range (clamped), bit 1 a token named an expert twice
    uint8_t *ws = nullptr;
    // single-token fused path (all matrices IQ2_XXS, shapes the fused kernel tiles)
    bool fused = false;
    // mixed-precision layouts (gate/up IQ2_XXS, IQ2_XS or IQ1_M, other matrices of other types): the routed gate/up matrices
    // are packed for the MFMA gate/up kernel, the down matrices stay raw GGUF rows; one token at a time
    bool mixed = false;
    uint64_t packed_stride = 0;              // bytes between experts in `packed`
    bool packed_gu() const { return fused || mixed; }
    // every path of an all-IQ2_XXS handle of these shapes reads the packed copies: the raw GGUF rows of the routed experts only pass
    // through a staging buffer at upload
    // So do the mixed layouts whose batches run as expert slices, when every size they can be given has kernels on the packed copies:
    // one token (packed gate | up, word- or stream-packed down), 2..8 tokens (slices), 9..16 (slices behind the own router, two small
    // batches or tiles with a caller's routing), larger chunks only
    // with the tile-major copies (a handle made for more than 16 tokens on a shape without tile kernels keeps the raw rows for the
    // raw-row kernels). Any kernel that would read raw rows on such a handle is refused on the host (raw_rows below).
    bool keep_raw() const {
        if (fused && cfg.hidden / 512u <= 4u) return false;
        if (mixed_slices && (cfg.max_tokens <= 2u * kSlice || (sliced_words() ? tiles_resident() : stream_tiles_resident()))) return false;
        return true;
    }
    // all-IQ2_XXS layers of the shapes whose chunks run on the tile-major copies read their down matrices from the column-sliced copy (one
    // token, small batches) or the tile-major one (chunks): the row-major packed down matrices are not kept (they pass through a second
    // staging buffer on their way to the tile-major copy)
    bool rowmajor_down() const { return !(fused && cfg.ffn <= 512u && cfg.hidden / 512u <= 4u); }
    uint8_t *stage_down = nullptr;           // row-major packed down matrices of kStageExperts experts, source of their tile-major copy
    uint8_t *stage = nullptr;                // upload staging for handles that do not keep the raw rows: kStageExperts slots
    static constexpr uint32_t kStageExperts = 64u;
    // handles that can be given chunks keep a tile-major copy for the prefill kernels that hold a tile's activations in registers
    // larger chunks take the router as a tiled f32 product (a quantised router through its f32 copy)
    // (below 40 tokens the f32 rows are quicker one token per grid layer - 12.1 against 14.0 us at 32 tokens, 14.4 against 13.8 at 40:
    // 32 x 32 tiles leave most of the chip idle there)
    bool tiled_router(uint32_t ntok) const { return packed_gu() && ntok >= 40u && (cfg.router_type == T_F32 || mixed); }
    uint64_t tiled_stride() const { return fused ? expert_stride : packed_stride; }      // bytes between experts in `tiled`
    bool tiles_resident() const { return packed_gu() && gu_type == T_IQ2_XXS && cfg.max_tokens > 8u && cfg.ffn <= 512u && cfg.hidden / 512u <= 4u; }
    // a chunk on a mixed layout: the routed gate/up matrices (packed IQ2_XXS) run on the prefill tiles, the rest on raw rows
    bool mixed_chunk(uint32_t ntok) const { return mixed && ntok > 8u && tiles_resident(); }
    uint64_t words_down_stride() const {
        return ((dn_type == T_IQ3_S ? iq3s_words_bytes(cfg.hidden, cfg.ffn) : packed_matrix_bytes(dn_type, cfg.hidden, cfg.ffn)) + 255u) & ~255ull;
    }
    uint64_t tiled_down_stride() const { return ((uint64_t)cfg.hidden * (cfg.ffn / 32u) * 16u + (uint64_t)cfg.hidden * (cfg.ffn / 256u) * 2u + 255u) & ~255ull; }
    // the one-launch router kernels (logits of every expert + the shared expert's gate logit, optional residual + norm) and the
    // one-wave selection serve every layout whose router they tile; the per-row GEMV + generic selection are what is left
    bool fast_route() const {
        const uint32_t nv = cfg.hidden / 256u;
        return packed_gu() || cfg.router_type == T_Q6_K || (cfg.router_type == T_F32 && (nv == 2u || nv == 4u || nv == 8u || nv == 16u));
    }
    void *xh = nullptr, *xl = nullptr;       // fp16 [hidden] each
    int *xexp = nullptr;
    bool skip_select = false;                // forward(): the gate/up kernel selects, route() skips its own selection
    bool shared_gu_ready = false;            // the router launch of this forward() has left the shared expert's gate / up products in `act`
    // batched path (ntok > 1): pairs grouped by expert
    uint32_t *uid = nullptr, *expert_start = nullptr, *pair_token = nullptr, *tok_pair = nullptr, *n_unique = nullptr;
    uint32_t *tile_group = nullptr, *tile_pair0 = nullptr, *tile_n = nullptr, *n_tiles = nullptr;      // prefill tiles
    void *group_mem = nullptr;               // handles that take more than 512 tokens: scratch of the pair sort by many workgroups
    GroupScratch group_scratch{};
    const GroupScratch *group_scratch_ptr() const { return group_mem ? &group_scratch : nullptr; }
    float *pair_weight = nullptr, *tmp = nullptr, *sh_tmp = nullptr;
    // chunks on mixed layouts: the shared expert's dense products (x -> sh_gu -> sh_act -> sh_tmp) run on a stream of their own beside
    // the routed experts' tile kernels, which leave most of the machine's issue slots free; forked and joined with events
    float *sh_gu = nullptr;                  // [max_tokens][2 ffn]
    hipStream_t side = nullptr;
    hipEvent_t ev_fork = nullptr, ev_join = nullptr;
    void *act_h = nullptr, *act_l = nullptr; // fp16 [top_k + 1][ffn] each
    int *act_exp = nullptr;                  // [top_k + 1][ffn / 32]

    // mixed layouts whose batches of 2..8 tokens run as expert slices: gate/up packed IQ2_XXS, down IQ3_S (column-sliced words), the shared
    // expert from its dense f32 copies, an f32 router (or the f32 copy of a quantised one) in the launch that leaves the shared gate | up products;
    // or every routed matrix IQ2_XS, or every one IQ1_M (gate | up as row-major streams, the down streams once more column-sliced)
    bool mixed_slices = false;
    // ... whose IQ3_S down matrices are kept column-sliced only (the one-token kernel reads that copy too)
    bool sliced_words() const { return mixed_slices && dn_type == T_IQ3_S; }
    // ... whose down matrices are IQ2_XS / IQ1_M streams: a column-sliced copy beside the row-major one
    bool sliced_streams() const { return mixed_slices && dn_type != T_IQ3_S; }
    // batches that run as expert slices per pass: 2..8 tokens and at most 128 pairs on mixed layouts (their first launch multiplies the
    // shared expert's gate | up rows for up to eight tokens), 2..16 tokens and at most 256 pairs on all-IQ2_XXS layers - 2..32 tokens and
    // 512 pairs behind the layer's own router (own_router: the selection launch sorts that many; a caller's routing is sorted by one more
    // workgroup of the launch that splits the activations, up to 256 pairs)
    static constexpr uint32_t kSmallMaxFused = 16u, kSmallMaxRouted = 32u, kSmallMaxGiven = 24u, kSmallMaxMixed = 32u;
    bool dense_routed = false;               // every layer has f32 copies of its router and of the shared expert's gate | up rows (set at creation)
    bool small_batch(uint32_t ntok, bool own_router = false) const {
        if (ntok < 2u || cfg.hidden / 512u > 4u) return false;
        if (fused) return ntok <= (own_router ? kSmallMaxRouted : kSmallMaxFused) && ntok * cfg.top_k <= (own_router ? 512u : 256u);
        // (mixed layouts behind their own router: the router launch is repeated per sixteen tokens, the selection launch sorts up to 512 pairs)
        if (own_router && ntok > 8u) return mixed_slices && dense_routed && ntok <= kSmallMaxMixed && ntok * cfg.top_k <= 512u;
        return mixed_slices && ntok <= 8u && ntok * cfg.top_k <= 128u && ntok * (cfg.top_k + 1u) <= 144u;
    }
    // ... with the layer's own router: on a mixed layout two tokens are quicker on the single-token kernels (three launches, the selection
    // inside the gate/up kernel) than as slices behind a selection + pair sort launch of their own (four): 30.7 against 32.7 us
    bool slices_after_router(uint32_t ntok) const { return small_batch(ntok, true) && (fused || ntok >= kGroupedMin); }
    // the same batches on a mixed layout run on the single-token kernels, one grid layer per token (tokens rarely share an
    // expert at these sizes, so reading a shared expert twice costs less than the pair sort and the per-pair kernels)
    bool small_batch_mixed(uint32_t ntok) const {
        return mixed && ntok >= 2u && ntok <= 8u && ntok * cfg.top_k <= 128u && ntok * (cfg.top_k + 1u) <= 144u && cfg.hidden / 512u <= 4u;
    }
    // from kGroupedMin tokens on such a batch is grouped by expert instead when its formats allow (packed IQ2_XXS gate/up on the batched
    // MFMA kernel, built-in down types on the batched raw-row kernel): every distinct expert is read once. Needs the router launch of the
    // same forward() for the shared expert's gate / up products.
    static constexpr uint32_t kGroupedMin = 3u;
    bool grouped_mixed(uint32_t ntok, uint32_t from = kGroupedMin) const {
        const uint32_t rbd = (cfg.ffn / 256u) * block_bytes(dn_type), rbs = (cfg.ffn / 256u) * block_bytes(sh_dn_type);
        const bool words = (dn_type == T_IQ3_S || dn_type == T_IQ2_XS || dn_type == T_IQ1_M) && cfg.ffn <= 1024u;      // then the layers hold a packed down copy
        return small_batch_mixed(ntok) && ntok >= from && (words || cfg.ffn <= 768u) &&
               (words || (quant_supported(dn_type) && (8u * rbd) % 16u == 0u && (8u * rbs) % 16u == 0u && (2u * gate_bytes) % 16u == 0u && (2u * sh_gate_bytes) % 16u == 0u));
    }
    // a chunk on a layout whose experts are IQ2_XS / IQ1_M: the tile kernels on the row-major streams of the routed matrices, the shared
    // expert and the router as dense f32 products
    bool stream_chunk(uint32_t ntok) const { return ntok > 8u && stream_tiles_resident(); }
    // ... such a handle keeps tile-major copies of the gate | up streams (`tiled`) and of the down streams (`tiled_down`)
    bool stream_tiles_resident() const {
        const bool gu_cb = gu_type == T_IQ2_XS || gu_type == T_IQ1_M, dn_cb = dn_type == T_IQ2_XS || dn_type == T_IQ1_M;
        return mixed && gu_cb && dn_cb && (cfg.ffn == 256u || cfg.ffn == 512u) && cfg.hidden / 512u <= 4u && cfg.max_tokens > 8u;
    }
    // a chunk on a mixed layout that has no tile kernels (ffn > 512, or IQ2_XS / IQ1_M gate/up beside another down format) runs as slices
    // of 8 tokens on the grouped small-batch kernels, far ahead of the generic per-pair kernels on raw rows
    static constexpr uint32_t kSlice = 8u;
    // So does every layout from 9 to 16 tokens: two small batches are quicker than one chunk, whose tile kernels leave most workgroups
    // without work at that size.
    bool sliced(uint32_t ntok) const {
        if (ntok <= kSlice || small_batch(ntok, true)) return false;      // (one small batch: up to 32 tokens behind the layer's own router)
        if (ntok <= 2u * kSlice && (small_batch(kSlice) || grouped_mixed(kSlice))) return true;
        return mixed && !tiles_resident() && !stream_chunk(ntok) && grouped_mixed(kSlice);
    }
    // the workspace entries a caller can read back (redhip_moe_last_route) of the slice that starts at token t0 sit at their place in the chunk
    void shift_route_outputs(int64_t t0) {
        ids += t0 * (int64_t)cfg.top_k;
        weights += t0 * (int64_t)cfg.top_k;
        logits += t0 * (int64_t)(cfg.n_expert + 1u);
    }
    // every batch size runs on the packed layout when the layer has one (decode kernel, small-batch kernels, prefill tiles)
    bool packed_path(uint32_t ntok) const { return (fused && (ntok == 1u || small_batch(ntok) || cfg.hidden / 512u <= 4u)) || (mixed && ntok == 1u); }
    ExpertSet routed(uint32_t l) const { return ExpertSet{layers[l].experts, expert_stride, gate_bytes, gate_bytes, gu_type, dn_type}; }
    ExpertSet shared(uint32_t l) const { return ExpertSet{layers[l].shared, 0, sh_gate_bytes, sh_gate_bytes, sh_gu_type, sh_dn_type}; }
};

Moe *moe_of(redhip_moe_t h) { return static_cast<Moe *>(h); }

// the raw GGUF rows of a layer's routed experts, for the kernels that read them; nullptr + message on a handle that keeps none
const uint8_t *raw_rows(const Moe *m, uint32_t layer) {
    const uint8_t *p = m->layers[layer].experts;
    if (!p) moe_err("internal: this handle keeps no raw rows of its routed experts, and a kernel that reads them was chosen (layer %u)", layer);
    return p;
}

size_t align256(size_t n) { return (n + 255u) & ~(size_t)255u; }

bool check_layer(Moe *m, uint32_t layer) {
    if (!m) { moe_err("null MoE handle"); return false; }
    if (layer >= m->cfg.n_layer) { moe_err("layer %u out of range (%u layers)", layer, m->cfg.n_layer); return false; }
    return true;
}

__global__ __launch_bounds__(256) void scalar_gate_kernel(const float *gate_inp, const float *x, uint32_t hidden, float *scalar) {
    __shared__ double red[4];
    const float *xt = x + (uint64_t)blockIdx.x * hidden;
    double acc = 0.0;
    for (uint32_t i = threadIdx.x; i < hidden; i += 256u) acc += (double)gate_inp[i] * (double)xt[i];
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if ((threadIdx.x & 63u) == 0u) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0u) scalar[blockIdx.x] = (float)(1.0 / (1.0 + exp(-((red[0] + red[1]) + (red[2] + red[3])))));
}

// resid = x + branch, xn = resid * rsqrt(mean(resid^2) + eps) * w (native/redlite_native_engine_cpu.c:418-424); one workgroup per
// token. Used when the router kernel of the path cannot normalise on the fly.
__global__ __launch_bounds__(256) void resid_rms_kernel(const float *x, const float *branch, const float *w, float eps, uint32_t hidden, float *xn) {
    __shared__ double red[4];
    const uint64_t base = (uint64_t)blockIdx.x * hidden;
    double ss = 0.0;
    for (uint32_t i = threadIdx.x; i < hidden; i += 256u) { const float v = x[base + i] + branch[base + i]; ss += (double)v * v; }
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if ((threadIdx.x & 63u) == 0u) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = (float)(1.0 / sqrt(((red[0] + red[1]) + (red[2] + red[3])) / (double)hidden + (double)eps));
    for (uint32_t i = threadIdx.x; i < hidden; i += 256u) xn[base + i] = ((x[base + i] + branch[base + i]) * inv) * w[i];
}

// The shared expert of a chunk on a mixed layout as dense f32 products (gate | up, SwiGLU, down) on the side stream: forked from s here,
// joined by join_shared_dense before the combine. Reads x, writes sh_gu, sh_act, sh_tmp, which nothing on s touches in between.
int fork_shared_dense(Moe *m, const Layer &L, const float *x, uint32_t ntok, hipStream_t s) {
    const redhip_moe_config &c = m->cfg;
    HIP_OK(hipEventRecord(m->ev_fork, s), "fork event");
    HIP_OK(hipStreamWaitEvent(m->side, m->ev_fork, 0), "fork wait");
    prof_set_stage(ST_BATCH_GATEUP);
    HIP_OK(launch_f32_tiles(L.dense_gu, nullptr, x, ntok, c.hidden, 2u * c.ffn, m->sh_gu, 2u * c.ffn, nullptr, nullptr, nullptr, m->side), "shared gate/up tiles");
    HIP_OK(launch_swiglu_rows(m->sh_gu, 2u * c.ffn, ntok, c.ffn, m->sh_act, m->side), "shared SwiGLU");
    prof_set_stage(ST_BATCH_DOWN);
    HIP_OK(launch_f32_tiles(L.dense_down, nullptr, m->sh_act, ntok, c.ffn, c.hidden, m->sh_tmp, c.hidden, nullptr, nullptr, nullptr, m->side), "shared down tiles");
    HIP_OK(hipEventRecord(m->ev_join, m->side), "join event");
    return 1;
}
int join_shared_dense(Moe *m, hipStream_t s) {
    HIP_OK(hipStreamWaitEvent(s, m->ev_join, 0), "join wait");
    return 1;
}

// select_here: the gate/up kernel selects the experts from m->logits itself (ids / weights are then outputs)
// grouped: the pair sort of (ids, weights) is already in the workspace
int experts_enqueue(Moe *m, uint32_t layer, const float *x, uint32_t ntok, const uint32_t *ids, const float *weights,
                    float *out, hipStream_t s, bool select_here = false, bool grouped = false) {
    const redhip_moe_config &c = m->cfg;
    // select_here && grouped: selection and pair sort both happen inside the batched gate/up kernel, from m->logits
    const BatchSelect bsel{m->logits, c.n_expert, m->ids, m->weights, m->scalar};
    const BatchSelect *in_batch = select_here && grouped ? &bsel : nullptr;
    if (m->mixed_slices && m->small_batch(ntok, true) && grouped) {     // pairs sorted (with their pass list) by the launch before; the shared gate | up products are in m->act
        if (select_here || !m->shared_gu_ready) { moe_err("internal: a small batch reached the expert slices without its routing or the shared expert's products"); return 0; }
        const Layer &L = m->layers[layer];
        HIP_OK(launch_batch_slices(L.packed, m->packed_stride, L.down_cm, m->down_cm_stride(), nullptr, nullptr, m->pass_list, m->n_pass, weights, m->scalar,
                                   m->xh, m->xl, m->xexp, m->partial, out, c.hidden, c.ffn, c.top_k, ntok, s, m->act, L.dense_down,
                                   m->sliced_streams() ? m->dn_type : 0u, m->sliced_streams() ? m->dn_grid : nullptr), "batched expert slice launch");
        prof_set_stage(ST_OTHER);
        return 1;
    }
    if (m->grouped_mixed(ntok, grouped ? 2u : Moe::kGroupedMin) && m->shared_gu_ready) {      // xh / xl / xexp / scalar and the shared gate | up products (m->act) come from the router launch
        const Layer &L = m->layers[layer];
        if (!grouped) {
            prof_set_stage(ST_GROUP);
            HIP_OK(launch_group_pairs(ids, weights, ntok, c.top_k, c.n_expert, m->uid, m->expert_start, m->pair_token, m->pair_weight,
                                      m->tok_pair, m->n_unique, s), "grouping launch");
        }
        if (!L.words_down && !raw_rows(m, layer)) return 0;          // (the batched down kernel reads the packed copy when there is one)
        HIP_OK(launch_batch_mixed(m->gu_type, m->gu_grid, L.packed, m->packed_stride, m->act, m->dn_type, m->dn_grid, m->sh_dn_type, L.experts ? L.experts + 2u * m->gate_bytes : nullptr, m->expert_stride,
                                  L.shared + 2u * m->sh_gate_bytes, L.words_down, m->words_down_stride(), L.dense_down, m->uid, m->expert_start, m->pair_token, m->n_unique, m->pair_weight, m->tok_pair,
                                  m->scalar, m->xh, m->xl, m->xexp, m->act_h, m->act_l, m->act_exp, out, c.hidden, c.ffn, c.top_k, ntok, c.n_expert, s, in_batch),
               "grouped mixed batch launch");
        prof_set_stage(ST_OTHER);
        return 1;
    }
    if (ntok > 1u && !m->small_batch_mixed(ntok)) {       // group the (token, expert) pairs by expert, run each distinct expert once over its tokens
        const uint32_t P = ntok * c.top_k, n_groups = P < c.n_expert ? P : c.n_expert;
        const ExpertSet ex = m->routed(layer), sh = m->shared(layer);
        const Layer &Ld = m->layers[layer];
        const bool stream_tiles = m->stream_chunk(ntok) && Ld.tiled && Ld.tiled_down && Ld.dense_gu && m->side;
        // the shared expert as dense f32 products on the fp32 matrix units, started before the pair sort (one workgroup on an idle machine;
        // the many-workgroup sort of a large chunk then queues behind the dense tiles - 73 against 22 us at 2048 tokens - but started
        // behind the sort the dense products slow the down tiles by more: 787 against 760 us per chunk)
        const bool dense_shared = (stream_tiles || (m->mixed_chunk(ntok) && Ld.dense_gu && m->side));
        if (dense_shared && !fork_shared_dense(m, Ld, x, ntok, s)) return 0;
        // the pair sort also writes the tile lists of the tile kernels that follow (all-IQ2_XXS layers: with the shared expert's tiles)
        const bool tile_path = !m->small_batch(ntok) && (m->packed_path(ntok) || stream_tiles || m->mixed_chunk(ntok));
        const TileLists tl{m->tile_group, m->tile_pair0, m->tile_n, m->n_tiles, prefill_tile_bound(ntok, c.top_k, c.n_expert), m->packed_path(ntok) ? ntok : 0u};
        const bool tiles_built = !grouped && tile_path;
        if (!grouped) {
            prof_set_stage(ST_GROUP);
            HIP_OK(launch_group_pairs(ids, weights, ntok, c.top_k, c.n_expert, m->uid, m->expert_start, m->pair_token, m->pair_weight,
                                      m->tok_pair, m->n_unique, s, tile_path ? &tl : nullptr, m->group_scratch_ptr()), "grouping launch");
        }
        if (m->small_batch(ntok, true) && grouped && !select_here) {     // routing sorted (with its pass list) by the prep or the selection launch: expert slices per pass
            const Layer &L = m->layers[layer];
            HIP_OK(launch_batch_slices(L.packed, m->packed_stride, L.down_cm, m->down_cm_stride(), L.shared_packed, L.shared_down_cm, m->pass_list, m->n_pass,
                                       weights, m->scalar, m->xh, m->xl, m->xexp, m->partial, out, c.hidden, c.ffn, c.top_k, ntok, s), "batched expert slice launch");
            prof_set_stage(ST_OTHER);
            return 1;
        }
        if (m->small_batch(ntok)) { moe_err("internal: a small batch reached the expert kernels without its pass list"); return 0; }
        if (m->packed_path(ntok)) {     // prefill chunk: tiles of 16 pairs per expert on the MFMA units
            const Layer &L = m->layers[layer];
            HIP_OK(launch_prefill_packed(L.packed, m->expert_stride, L.shared_packed, L.tiled, L.shared_tiled, m->uid, m->expert_start, m->pair_token, m->n_unique,
                                         m->tile_group, m->tile_pair0, m->tile_n, m->n_tiles, m->xh, m->xl, m->xexp, m->act_h, m->act_l,
                                         m->act_exp, m->tmp, m->sh_tmp, c.hidden, c.ffn, c.top_k, ntok, c.n_expert, s, tiles_built), "prefill launch");
            prof_set_stage(ST_BATCH_COMBINE);
            HIP_OK(launch_batch_combine(m->tmp, m->pair_weight, m->tok_pair, ntok, c.top_k, m->sh_tmp, m->scalar, c.hidden, out, s), "batched combine launch");
            prof_set_stage(ST_OTHER);
            return 1;
        }
        if (stream_tiles) {
            const Layer &L = Ld;
            prof_set_stage(ST_BATCH_GATEUP);
            HIP_OK(launch_prefill_streams(m->gu_type, m->gu_grid, L.tiled, m->packed_stride, m->dn_type, m->dn_grid, L.tiled_down, m->words_down_stride(), m->uid,
                                          m->expert_start, m->pair_token, m->n_unique, m->tile_group, m->tile_pair0, m->tile_n, m->n_tiles, m->xh, m->xl, m->xexp,
                                          m->act_h, m->act_l, m->act_exp, m->tmp, c.hidden, c.ffn, c.top_k, ntok, c.n_expert, s, tiles_built), "stream tile launch");
            if (!join_shared_dense(m, s)) return 0;
            prof_set_stage(ST_BATCH_COMBINE);
            HIP_OK(launch_batch_combine(m->tmp, m->pair_weight, m->tok_pair, ntok, c.top_k, m->sh_tmp, m->scalar, c.hidden, out, s), "batched combine launch");
            prof_set_stage(ST_OTHER);
            return 1;
        }
        prof_set_stage(ST_BATCH_GATEUP);
        const bool tiled_down = m->mixed_chunk(ntok) && m->layers[layer].tiled_down;      // then the activations stay fp16 halves for the IQ3_S tile kernel
        if (!(m->mixed_chunk(ntok) && tiled_down) && !raw_rows(m, layer)) return 0;       // (the per-pair kernels below read raw rows)
        if (m->mixed_chunk(ntok))      // xh / xl / xexp come from the router kernel or the prep kernel
            HIP_OK(launch_prefill_gateup_tiled(m->layers[layer].tiled, m->packed_stride, m->uid, m->expert_start, m->pair_token, m->n_unique, m->tile_group,
                                               m->tile_pair0, m->tile_n, m->n_tiles, m->xh, m->xl, m->xexp, tiled_down ? nullptr : m->act, m->act_h, m->act_l,
                                               m->act_exp, c.hidden, c.ffn, c.top_k, ntok, c.n_expert, s, tiles_built), "tiled gate/up launch");
        else
            HIP_OK(launch_batch_gateup(ex, m->uid, m->expert_start, m->pair_token, m->n_unique, n_groups, P, c.hidden, c.ffn, x, m->act, s), "batched gate/up launch");
        prof_set_stage(ST_BATCH_GATEUP);
        if (!dense_shared) {
            HIP_OK(launch_batch_gateup(sh, nullptr, nullptr, nullptr, nullptr, 1u, ntok, c.hidden, c.ffn, x, m->sh_act, s), "batched shared gate/up launch");
        }
        prof_set_stage(ST_BATCH_DOWN);
        if (tiled_down)
            HIP_OK(launch_prefill_down_iq3s(Ld.tiled_down, m->tiled_down_stride(), m->uid, m->n_unique, m->tile_group, m->tile_pair0, m->tile_n, m->n_tiles,
                                            m->act_h, m->act_l, m->act_exp, m->tmp, c.hidden, c.ffn, c.top_k, ntok, c.n_expert, s), "tiled IQ3_S down launch");
        else
            HIP_OK(launch_batch_down(ex, m->uid, m->expert_start, m->n_unique, n_groups, P, c.hidden, c.ffn, m->act, m->tmp, s), "batched down launch");
        prof_set_stage(ST_BATCH_DOWN);
        if (dense_shared) {
            if (!join_shared_dense(m, s)) return 0;
        } else
            HIP_OK(launch_batch_down(sh, nullptr, nullptr, nullptr, 1u, ntok, c.hidden, c.ffn, m->sh_act, m->sh_tmp, s), "batched shared down launch");
        prof_set_stage(ST_BATCH_COMBINE);
        HIP_OK(launch_batch_combine(m->tmp, m->pair_weight, m->tok_pair, ntok, c.top_k, m->sh_tmp, m->scalar, c.hidden, out, s), "batched combine launch");
        prof_set_stage(ST_OTHER);
        return 1;
    }
    if (m->fused && ntok == 1u) {    // expert slices + their sum; xh / xl (and the scalar gate of a caller's routing) come from the router kernel or the prep kernel
        const Layer &L = m->layers[layer];
        HIP_OK(launch_expert_slices(L.packed, m->packed_stride, L.down_cm, m->down_cm_stride(), L.shared_packed, L.shared_down_cm, select_here ? m->logits : nullptr,
                                    ids, weights, m->scalar, m->ids, m->weights, m->scalar, m->xh, m->xl, m->xexp, m->partial, out, c.hidden, c.ffn, c.n_expert,
                                    c.top_k, s), "expert slice launch");
        prof_set_stage(ST_OTHER);
        return 1;
    }
    if (m->mixed_slices && ntok == 1u && m->shared_gu_ready && m->layers[layer].dense_down) {
        // one token on a mixed layout whose small batches run as slices: the same slices, the down matrices from their column-sliced copy, the
        // shared expert from its products (m->act, left by the router launch) and the dense copy of its down matrix
        const Layer &L = m->layers[layer];
        HIP_OK(launch_expert_slices(L.packed, m->packed_stride, L.down_cm, m->down_cm_stride(), nullptr, nullptr, select_here ? m->logits : nullptr,
                                    ids, weights, m->scalar, m->ids, m->weights, m->scalar, m->xh, m->xl, m->xexp, m->partial, out, c.hidden, c.ffn, c.n_expert,
                                    c.top_k, s, m->act, L.dense_down, m->sliced_streams() ? m->dn_type : 0u, m->sliced_streams() ? m->dn_grid : nullptr), "expert slice launch");
        prof_set_stage(ST_OTHER);
        return 1;
    }
    if (m->packed_gu()) {    // xh / xl / scalar come from the router kernel or the prep kernel
        const Layer &L = m->layers[layer];
        prof_set_stage(ST_GATEUP);
        HIP_OK(launch_gateup_select(L.packed, m->packed_stride, L.shared_packed, L.shared, x, m->shared_gu_ready ? m->act : nullptr,
                                    select_here ? m->logits : nullptr, ids, m->ids,
                                    m->weights, m->scalar, m->xh, m->xl, m->xexp, m->act_h, m->act_l, m->act_exp, c.hidden, c.ffn, c.n_expert,
                                    c.top_k, s, ntok, m->gu_type, m->gu_grid), "gate/up launch");      // ntok > 1: a small batch on a mixed layout, one grid layer per token
        prof_set_stage(ST_DOWN_COMBINE);
        if ((L.words_down || m->sliced_words()) && L.dense_down)      // (layers whose small batches run as slices keep their IQ3_S words column-sliced only)
            HIP_OK(launch_down_combine_words(m->dn_type, m->dn_grid, m->sliced_words() ? L.down_cm : L.words_down, m->words_down_stride(), L.dense_down,
                                             select_here ? m->ids : ids, select_here ? m->weights : weights,
                                             m->scalar, m->act_h, m->act_l, m->act_exp, out, c.hidden, c.ffn, c.top_k, s, ntok, m->sliced_words()), "down/combine launch");
        else if (!raw_rows(m, layer))
            return 0;
        else
            HIP_OK(launch_down_combine_raw(m->dn_type, m->sh_dn_type, L.experts + 2u * m->gate_bytes, m->expert_stride, L.shared + 2u * m->sh_gate_bytes,
                                           select_here ? m->ids : ids, select_here ? m->weights : weights, m->scalar, m->act_h, m->act_l,
                                           m->act_exp, out, c.hidden, c.ffn, c.top_k, s, ntok, m->dn_grid, L.dense_down), "down/combine launch");
        prof_set_stage(ST_OTHER);
        return 1;
    }
    if (!raw_rows(m, layer)) return 0;
    const ExpertSet ex = m->routed(layer), sh = m->shared(layer);
    prof_set_stage(ST_GATEUP);
    HIP_OK(launch_moe_gateup(ex, ids, c.top_k, c.hidden, c.ffn, x, m->act, s), "routed gate/up launch");
    prof_set_stage(ST_SHARED_GATEUP);
    HIP_OK(launch_moe_gateup(sh, nullptr, 1u, c.hidden, c.ffn, x, m->sh_act, s), "shared gate/up launch");
    prof_set_stage(ST_DOWN_COMBINE);
    HIP_OK(launch_moe_down_combine(ex, ids, weights, c.top_k, sh, m->scalar, c.hidden, c.ffn, m->act, m->sh_act, out, s), "down/combine launch");
    prof_set_stage(ST_OTHER);
    return 1;
}

// a small batch on an all-IQ2_XXS layer behind the router launch: selection + pair sort (one launch), expert slices per pass, their sum
int select_group_slices(Moe *m, uint32_t layer, const float *x, uint32_t ntok, float *out, hipStream_t s) {
    const redhip_moe_config &c = m->cfg;
    const GroupJob job{nullptr, nullptr, ntok, c.top_k, c.n_expert, m->uid, m->expert_start, m->pair_token, m->pair_weight, m->tok_pair, m->n_unique, nullptr,
                       m->pass_list, m->n_pass};
    prof_set_stage(ST_ROUTE_SELECT);
    HIP_OK(launch_select_group(m->logits, ntok, c.n_expert, c.top_k, m->ids, m->weights, m->scalar, job, s), "selection + pair sort launch");
    return experts_enqueue(m, layer, x, ntok, m->ids, m->weights, out, s, false, true);
}

}  // namespace

extern "C" {

uint32_t redhip_moe_abi_version(void) { return 1u; }
const char *redhip_moe_last_error(void) { return g_moe_error[0] ? g_moe_error : "unknown redhip MoE error"; }

redhip_moe_t redhip_moe_create(const redhip_moe_config *cfg) {
    g_moe_error[0] = '\0';
    if (!cfg) { moe_err("null MoE config"); return nullptr; }
    const redhip_moe_config c = *cfg;
    const uint32_t gu = word_gate_up(c.expert_type_word), dn = word_down(c.expert_type_word);
    const uint32_t sgu = word_gate_up(c.shared_type_word), sdn = word_down(c.shared_type_word);
    if (!c.hidden || c.hidden % 256u || !c.ffn || c.ffn % 256u || !c.n_expert || c.n_expert > 1024u || !c.top_k || c.top_k > 16u ||
        c.top_k > c.n_expert || !c.n_layer || !c.max_tokens) {
        moe_err("invalid MoE shape hidden=%u ffn=%u experts=%u top_k=%u layers=%u max_tokens=%u", c.hidden, c.ffn, c.n_expert, c.top_k, c.n_layer, c.max_tokens);
        return nullptr;
    }
    if (!pool_quant_supported(gu) || !pool_quant_supported(dn) || !quant_supported(sgu) || !quant_supported(sdn) ||
        (c.router_type != T_F32 && c.router_type != T_Q6_K) || (c.expert_type_word >> 16) || (c.shared_type_word >> 16)) {
        moe_err("unsupported MoE types router=%u experts=0x%x shared=0x%x", c.router_type, c.expert_type_word, c.shared_type_word);
        return nullptr;
    }
    if (!caller_grid_present(gu) || !caller_grid_present(dn)) {
        moe_err("IQ2_XS / IQ1_M experts decode through the caller's codebooks: call redhip_set_codebooks first");
        return nullptr;
    }
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { moe_err("no HIP device available"); return nullptr; }
    Moe *m = new Moe();
    m->cfg = c;
    m->gu_type = gu; m->dn_type = dn; m->sh_gu_type = sgu; m->sh_dn_type = sdn;
    m->gate_bytes = (uint64_t)c.ffn * pool_row_bytes(gu, c.hidden);
    m->down_bytes = (uint64_t)c.hidden * pool_row_bytes(dn, c.ffn);
    m->expert_stride = align256(2u * m->gate_bytes + m->down_bytes);
    m->sh_gate_bytes = (uint64_t)c.ffn * row_bytes(sgu, c.hidden);
    m->sh_down_bytes = (uint64_t)c.hidden * row_bytes(sdn, c.ffn);
    m->router_bytes = (uint64_t)c.n_expert * row_bytes(c.router_type, c.hidden);
    m->layers.resize(c.n_layer);
    // the one-token kernels of the packed paths give every slot (top_k routed + the shared expert) a wave of a 16-wave workgroup, and the mixed
    // ones keep the shared expert's gate | up products in the activation rows of two routed slots: other top_k run on the generic kernels
    const bool slots_fit = c.top_k + 1u <= 16u;
    m->fused = gu == T_IQ2_XXS && dn == T_IQ2_XXS && sgu == T_IQ2_XXS && sdn == T_IQ2_XXS && fused_iq2_supported(c.hidden, c.ffn) && slots_fit;
    // (the raw-row down kernel stages 8 rows per slot in LDS: keep that within the default 64 KB)
    // IQ2_XS / IQ1_M gate/up matrices have a packed form of their own (a shared expert beside them is Q6_K; the gate/up kernel keeps
    // their fp16 codebook in LDS next to the staged Q6_K rows: 32 KB for IQ1_M)
    const bool gu_codebook = gu == T_IQ2_XS || gu == T_IQ1_M;
    m->mixed = !m->fused && slots_fit && c.top_k >= 2u && (gu == T_IQ2_XXS || gu_codebook) && (sgu == T_Q6_K || (sgu == T_IQ2_XXS && !gu_codebook)) && fused_iq2_supported(c.hidden, c.ffn) &&
               (size_t)(c.top_k + 1u) * 8u * (c.ffn / 256u) * 210u + (dn == T_IQ1_M ? 17u * 1024u : dn == T_IQ2_XS ? 5u * 1024u : 0u) <= 64u * 1024u &&
               (sgu != T_Q6_K || (size_t)64u * (c.hidden / 256u) * 210u + (size_t)(c.hidden + c.hidden / 32u + c.hidden / 16u) * 4u <= (gu == T_IQ1_M ? 120u : 144u) * 1024u);
    {
        const uint32_t nv = c.hidden / 256u;
        // (a handle for one token at a time needs no second copy of IQ2_XS / IQ1_M down streams: only the slices read the column-sliced one)
        m->mixed_slices = m->mixed && ((gu == T_IQ2_XXS && dn == T_IQ3_S) || (gu_codebook && dn == gu && sgu == T_Q6_K)) && c.ffn <= 512u &&
                          c.hidden / 512u <= 4u && (nv == 2u || nv == 4u || nv == 8u || nv == 16u);
        m->dense_routed = m->mixed_slices;      // (every mixed layer gets f32 copies of its shared expert, and of its router unless that is f32 already)
    }
    m->pk_gate_bytes = packed_matrix_bytes(gu, c.ffn, c.hidden);
    m->packed_stride = m->fused && m->rowmajor_down() ? m->expert_stride : align256(2u * m->pk_gate_bytes);
    m->gu_grid = caller_grid_device(gu);
    m->dn_grid = caller_grid_device(dn);
    if (m->gu_grid || m->dn_grid) (void)set_caller_grids(nullptr, nullptr, m);      // bound to the tables the process holds now: they cannot change under this handle
    bool ok = true;
    for (uint32_t l = 0; l < c.n_layer && ok; ++l) {
        Layer &L = m->layers[l];
        const size_t small = align256(m->router_bytes) + align256(2u * m->sh_gate_bytes + m->sh_down_bytes) + align256(4u * c.hidden);
        uint8_t *p = nullptr;
        ok = hipMalloc(reinterpret_cast<void **>(&p), small) == hipSuccess &&
             (!m->keep_raw() || hipMalloc(reinterpret_cast<void **>(&L.experts), (size_t)c.n_expert * m->expert_stride) == hipSuccess);
        if (!ok) { if (p) (void)hipFree(p); break; }
        L.router = p;
        L.shared = p + align256(m->router_bytes);
        L.gate_inp = reinterpret_cast<float *>(L.shared + align256(2u * m->sh_gate_bytes + m->sh_down_bytes));
        m->resident += small + (m->keep_raw() ? (uint64_t)c.n_expert * m->expert_stride : 0u);
        if (m->packed_gu()) {
            const bool sh_packed = m->sh_gu_type == T_IQ2_XXS;       // otherwise the shared expert is read from its raw rows
            ok = hipMalloc(reinterpret_cast<void **>(&L.packed), (size_t)c.n_expert * m->packed_stride) == hipSuccess &&
                 (!sh_packed || hipMalloc(reinterpret_cast<void **>(&L.shared_packed), align256(2u * m->sh_gate_bytes + m->sh_down_bytes)) == hipSuccess);
            m->resident += (uint64_t)c.n_expert * m->packed_stride + (sh_packed ? align256(2u * m->sh_gate_bytes + m->sh_down_bytes) : 0u);
        }
        if (ok && m->fused) {
            ok = hipMalloc(reinterpret_cast<void **>(&L.down_cm), (size_t)c.n_expert * m->down_cm_stride()) == hipSuccess &&
                 hipMalloc(reinterpret_cast<void **>(&L.shared_down_cm), m->down_cm_stride()) == hipSuccess;
            m->resident += (uint64_t)(c.n_expert + 1u) * m->down_cm_stride();
        }
        if (ok && m->mixed) {
            const size_t rb = c.router_type == T_F32 ? 0u : (size_t)c.n_expert * c.hidden * 4u, gb = (size_t)2u * c.ffn * c.hidden * 4u, db = (size_t)c.hidden * c.ffn * 4u;
            float *d = nullptr;
            ok = hipMalloc(reinterpret_cast<void **>(&d), align256(rb) + align256(gb) + align256(db)) == hipSuccess;
            if (ok) {
                L.dense_router = rb ? d : nullptr;
                L.dense_gu = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(d) + align256(rb));
                L.dense_down = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(L.dense_gu) + align256(gb));
                m->resident += align256(rb) + align256(gb) + align256(db);
            }
        }
        if (ok && m->mixed_slices) {
            ok = hipMalloc(reinterpret_cast<void **>(&L.down_cm), (size_t)c.n_expert * m->down_cm_stride()) == hipSuccess;
            m->resident += (uint64_t)c.n_expert * m->down_cm_stride();
        }
        if (ok && m->mixed && !m->sliced_words() && (dn == T_IQ3_S || dn == T_IQ2_XS || dn == T_IQ1_M) && c.ffn <= 1024u) {
            ok = hipMalloc(reinterpret_cast<void **>(&L.words_down), (size_t)c.n_expert * m->words_down_stride()) == hipSuccess;
            m->resident += (uint64_t)c.n_expert * m->words_down_stride();
        }
        if (ok && m->mixed && m->tiles_resident() && dn == T_IQ3_S) {
            ok = hipMalloc(reinterpret_cast<void **>(&L.tiled_down), (size_t)c.n_expert * m->tiled_down_stride()) == hipSuccess;
            m->resident += (uint64_t)c.n_expert * m->tiled_down_stride();
        }
        if (ok && m->stream_tiles_resident()) {
            ok = hipMalloc(reinterpret_cast<void **>(&L.tiled), (size_t)c.n_expert * m->tiled_stride()) == hipSuccess &&
                 hipMalloc(reinterpret_cast<void **>(&L.tiled_down), (size_t)c.n_expert * m->words_down_stride()) == hipSuccess;
            m->resident += (uint64_t)c.n_expert * (m->tiled_stride() + m->words_down_stride());
        }
        if (ok && m->tiles_resident()) {
            ok = hipMalloc(reinterpret_cast<void **>(&L.tiled), (size_t)c.n_expert * m->tiled_stride()) == hipSuccess &&
                 (!m->fused || hipMalloc(reinterpret_cast<void **>(&L.shared_tiled), align256(2u * m->sh_gate_bytes + m->sh_down_bytes)) == hipSuccess);
            m->resident += (uint64_t)c.n_expert * m->tiled_stride() + (m->fused ? align256(2u * m->sh_gate_bytes + m->sh_down_bytes) : 0u);
        }
    }
    const size_t T = c.max_tokens;
    const size_t partial_tokens = m->fused ? Moe::kSmallMaxRouted : Moe::kSmallMaxMixed;      // the largest batch that runs as expert slices
    const size_t partial_bytes = m->fused || m->mixed_slices ? align256((size_t)(c.max_tokens < partial_tokens ? c.max_tokens : partial_tokens) * (c.top_k + 1u) * (c.ffn / 32u) * c.hidden * 4u) : 0u;
    const size_t ws_bytes = partial_bytes + align256(8u * 512u) + align256(4u) + align256(4u) + align256(T * c.hidden * 4u) + align256(T * (c.n_expert + 1u) * 4u) + 2u * align256(T * c.top_k * 4u) + align256(T * 4u) +
                            align256(T * c.top_k * c.ffn * 4u) + align256(T * c.ffn * 4u) +
                            2u * align256(2u * T * c.hidden) + align256(4u * T) + 2u * align256(2u * T * (c.top_k + 1u) * c.ffn) +
                            align256(4u * T * (c.top_k + 1u) * (c.ffn / 32u)) +
                            (T > 8u && m->mixed ? align256(8u * T * c.ffn) : 0u) +
                            (T > 1u ? 6u * align256(4u * (T * c.top_k + 2u)) + align256(4u * T * c.top_k * c.hidden) + align256(4u * T * c.hidden) +
                                          4u * align256(12u * (size_t)prefill_tile_bound(c.max_tokens, c.top_k, c.n_expert)) : 0u);      // (three tile lists)
    ok = ok && hipMalloc(reinterpret_cast<void **>(&m->ws), ws_bytes) == hipSuccess;
    if (!ok) {
        moe_err("failed to allocate resident MoE memory (%llu bytes so far)", (unsigned long long)m->resident);
        redhip_moe_destroy(m);
        return nullptr;
    }
    uint8_t *w = m->ws;
    m->status = reinterpret_cast<uint32_t *>(w); w += align256(4u);
    if (partial_bytes) { m->partial = reinterpret_cast<float *>(w); w += partial_bytes; }
    m->pass_list = reinterpret_cast<uint2 *>(w); w += align256(8u * 512u);
    m->n_pass = reinterpret_cast<uint32_t *>(w); w += align256(4u);
    m->xn = reinterpret_cast<float *>(w); w += align256(T * c.hidden * 4u);
    m->logits = reinterpret_cast<float *>(w); w += align256(T * (c.n_expert + 1u) * 4u);
    m->ids = reinterpret_cast<uint32_t *>(w); w += align256(T * c.top_k * 4u);
    m->weights = reinterpret_cast<float *>(w); w += align256(T * c.top_k * 4u);
    m->scalar = reinterpret_cast<float *>(w); w += align256(T * 4u);
    m->act = reinterpret_cast<float *>(w); w += align256(T * c.top_k * c.ffn * 4u);
    m->sh_act = reinterpret_cast<float *>(w); w += align256(T * c.ffn * 4u);
    m->xh = w; w += align256(2u * T * c.hidden);
    m->xl = w; w += align256(2u * T * c.hidden);
    m->xexp = reinterpret_cast<int *>(w); w += align256(4u * T);
    m->act_h = w; w += align256(2u * T * (c.top_k + 1u) * c.ffn);
    m->act_l = w; w += align256(2u * T * (c.top_k + 1u) * c.ffn);
    m->act_exp = reinterpret_cast<int *>(w); w += align256(4u * T * (c.top_k + 1u) * (c.ffn / 32u));
    if (T > 8u && m->mixed) {
        m->sh_gu = reinterpret_cast<float *>(w); w += align256(8u * T * c.ffn);
        if (hipStreamCreateWithFlags(&m->side, hipStreamNonBlocking) != hipSuccess || hipEventCreateWithFlags(&m->ev_fork, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&m->ev_join, hipEventDisableTiming) != hipSuccess) {
            moe_err("failed to create the side stream of the shared expert");
            redhip_moe_destroy(m);
            return nullptr;
        }
    }
    if (T > 1u) {
        const size_t pw = align256(4u * (T * c.top_k + 2u));
        m->uid = reinterpret_cast<uint32_t *>(w); w += pw;
        m->expert_start = reinterpret_cast<uint32_t *>(w); w += pw;
        m->pair_token = reinterpret_cast<uint32_t *>(w); w += pw;
        m->tok_pair = reinterpret_cast<uint32_t *>(w); w += pw;
        m->n_unique = reinterpret_cast<uint32_t *>(w); w += pw;
        m->pair_weight = reinterpret_cast<float *>(w); w += pw;
        m->tmp = reinterpret_cast<float *>(w); w += align256(4u * T * c.top_k * c.hidden);
        m->sh_tmp = reinterpret_cast<float *>(w); w += align256(4u * T * c.hidden);
        const size_t tw = align256(12u * (size_t)prefill_tile_bound(c.max_tokens, c.top_k, c.n_expert));
        m->tile_group = reinterpret_cast<uint32_t *>(w); w += tw;
        m->tile_pair0 = reinterpret_cast<uint32_t *>(w); w += tw;
        m->tile_n = reinterpret_cast<uint32_t *>(w); w += tw;
        m->n_tiles = reinterpret_cast<uint32_t *>(w);
    }
    if (hipMemset(m->ws, 0, ws_bytes) != hipSuccess) { moe_err("failed to clear the MoE workspace"); redhip_moe_destroy(m); return nullptr; }
    if (T > 512u) {
        const size_t gb = group_scratch_bytes(c.max_tokens, c.n_expert);
        if (hipMalloc(&m->group_mem, gb) != hipSuccess || hipMemset(m->group_mem, 0, gb) != hipSuccess) {
            moe_err("failed to allocate the pair sort scratch");
            redhip_moe_destroy(m);
            return nullptr;
        }
        m->group_scratch = group_scratch_at(m->group_mem, c.max_tokens, c.n_expert);
        m->resident += gb;
    }
    // first launches copy the codebooks to the device; do it here so that forward never synchronises
    if (launch_dequant_rows(T_F32, m->ws, 1u, 32u, m->logits, nullptr) != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
        moe_err("failed to initialise device codebooks");
        redhip_moe_destroy(m);
        return nullptr;
    }
    return m;
}

void redhip_moe_destroy(redhip_moe_t h) {
    Moe *m = moe_of(h);
    if (!m) return;
    (void)hipDeviceSynchronize();
    forget_caller_grids(m);
    for (Layer &L : m->layers) {
        if (L.router) (void)hipFree(L.router);
        if (L.experts) (void)hipFree(L.experts);
        if (L.packed) (void)hipFree(L.packed);
        if (L.shared_packed) (void)hipFree(L.shared_packed);
        if (L.down_cm) (void)hipFree(L.down_cm);
        if (L.shared_down_cm) (void)hipFree(L.shared_down_cm);
        if (L.dense_gu) (void)hipFree(L.dense_router ? L.dense_router : L.dense_gu);
        if (L.tiled) (void)hipFree(L.tiled);
        if (L.tiled_down) (void)hipFree(L.tiled_down);
        if (L.words_down) (void)hipFree(L.words_down);
        if (L.shared_tiled) (void)hipFree(L.shared_tiled);
    }
    if (m->ev_fork) (void)hipEventDestroy(m->ev_fork);
    if (m->ev_join) (void)hipEventDestroy(m->ev_join);
    if (m->side) (void)hipStreamDestroy(m->side);
    if (m->ws) (void)hipFree(m->ws);
    if (m->group_mem) (void)hipFree(m->group_mem);
    if (m->stage) (void)hipFree(m->stage);
    if (m->stage_down) (void)hipFree(m->stage_down);
    delete m;
}

uint64_t redhip_moe_resident_bytes(redhip_moe_t h) { return h ? moe_of(h)->resident : 0u; }

int redhip_moe_load_router(redhip_moe_t h, uint32_t layer, const void *weights, uint64_t bytes) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    if (!weights || bytes != m->router_bytes) { moe_err("router byte size mismatch: got %llu expected %llu", (unsigned long long)bytes, (unsigned long long)m->router_bytes); return 0; }
    HIP_OK(hipMemcpy(m->layers[layer].router, weights, (size_t)bytes, hipMemcpyDefault), "router upload");
    if (m->layers[layer].dense_router) {
        HIP_OK(launch_dequant_rows(m->cfg.router_type, m->layers[layer].router, m->cfg.n_expert, m->cfg.hidden, m->layers[layer].dense_router, nullptr), "router dequant");
        HIP_OK(hipStreamSynchronize(nullptr), "router dequant");
    }
    return 1;
}

int redhip_moe_load_shared(redhip_moe_t h, uint32_t layer, const float *gate_inp, const void *gate, uint64_t gate_bytes,
                           const void *up, uint64_t up_bytes, const void *down, uint64_t down_bytes) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    if (!gate_inp || !gate || !up || !down || gate_bytes != m->sh_gate_bytes || up_bytes != m->sh_gate_bytes || down_bytes != m->sh_down_bytes) {
        moe_err("shared expert byte size mismatch gate=%llu/%llu up=%llu/%llu down=%llu/%llu", (unsigned long long)gate_bytes,
                (unsigned long long)m->sh_gate_bytes, (unsigned long long)up_bytes, (unsigned long long)m->sh_gate_bytes,
                (unsigned long long)down_bytes, (unsigned long long)m->sh_down_bytes);
        return 0;
    }
    Layer &L = m->layers[layer];
    HIP_OK(hipMemcpy(L.gate_inp, gate_inp, 4u * (size_t)m->cfg.hidden, hipMemcpyDefault), "shared gate vector upload");
    HIP_OK(hipMemcpy(L.shared, gate, (size_t)gate_bytes, hipMemcpyDefault), "shared gate upload");
    HIP_OK(hipMemcpy(L.shared + gate_bytes, up, (size_t)up_bytes, hipMemcpyDefault), "shared up upload");
    HIP_OK(hipMemcpy(L.shared + 2u * gate_bytes, down, (size_t)down_bytes, hipMemcpyDefault), "shared down upload");
    if (L.dense_gu) {
        const redhip_moe_config &c = m->cfg;
        HIP_OK(launch_dequant_rows(m->sh_gu_type, L.shared, 2u * c.ffn, c.hidden, L.dense_gu, nullptr), "shared gate/up dequant");
        HIP_OK(launch_dequant_rows(m->sh_dn_type, L.shared + 2u * gate_bytes, c.hidden, c.ffn, L.dense_down, nullptr), "shared down dequant");
        HIP_OK(hipStreamSynchronize(nullptr), "shared dequant");
    }
    if (L.shared_packed) {
        const redhip_moe_config &c = m->cfg;
        HIP_OK(launch_repack_iq2xxs(L.shared, gate_bytes, 2u, c.ffn, c.hidden, false, L.shared_packed, gate_bytes, nullptr), "shared gate/up repack");
        if (m->fused) {
            HIP_OK(launch_repack_iq2xxs(L.shared + 2u * gate_bytes, 0u, 1u, c.hidden, c.ffn, false, L.shared_packed + 2u * gate_bytes, 0u, nullptr), "shared down repack");
            HIP_OK(launch_repack_iq2xxs(L.shared + 2u * gate_bytes, 0u, 1u, c.hidden, c.ffn, true, L.shared_down_cm, 0u, nullptr), "shared down column slices");
        }
        if (L.shared_tiled) {
            HIP_OK(launch_tile_packed(L.shared_packed, gate_bytes, 2u, c.ffn, c.hidden, L.shared_tiled, gate_bytes, nullptr), "shared gate/up tiling");
            HIP_OK(launch_tile_packed(L.shared_packed + 2u * gate_bytes, 0u, 1u, c.hidden, c.ffn, L.shared_tiled + 2u * gate_bytes, 0u, nullptr), "shared down tiling");
        }
        HIP_OK(hipStreamSynchronize(nullptr), "shared repack");
    }
    return 1;
}

static int stage_and_pack(Moe *m, uint32_t layer, uint32_t first, uint32_t count, uint8_t *dst, const uint8_t *gate, const uint8_t *up, const uint8_t *down);

int redhip_moe_load_experts(redhip_moe_t h, uint32_t layer, uint32_t first, uint32_t count, const void *gate, const void *up, const void *down) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    if (!gate || !up || !down || !count || first >= m->cfg.n_expert || count > m->cfg.n_expert - first) {
        moe_err("invalid expert range first=%u count=%u of %u", first, count, m->cfg.n_expert);
        return 0;
    }
    if (!m->keep_raw()) {           // through the staging buffer, a few experts at a time
        if (!m->stage) {
            HIP_OK(hipMalloc(reinterpret_cast<void **>(&m->stage), (size_t)Moe::kStageExperts * m->expert_stride), "staging allocation");
            m->resident += (uint64_t)Moe::kStageExperts * m->expert_stride;
        }
        if (!m->stage_down && !m->rowmajor_down() && m->tiles_resident()) {
            HIP_OK(hipMalloc(reinterpret_cast<void **>(&m->stage_down), (size_t)Moe::kStageExperts * m->down_cm_stride()), "down staging allocation");
            m->resident += (uint64_t)Moe::kStageExperts * m->down_cm_stride();
        }
        for (uint32_t done = 0; done < count; done += Moe::kStageExperts) {
            const uint32_t n = count - done < Moe::kStageExperts ? count - done : Moe::kStageExperts;
            if (!stage_and_pack(m, layer, first + done, n, m->stage, static_cast<const uint8_t *>(gate) + (uint64_t)done * m->gate_bytes,
                                static_cast<const uint8_t *>(up) + (uint64_t)done * m->gate_bytes, static_cast<const uint8_t *>(down) + (uint64_t)done * m->down_bytes))
                return 0;
        }
        return 1;
    }
    return stage_and_pack(m, layer, first, count, m->layers[layer].experts + (uint64_t)first * m->expert_stride, static_cast<const uint8_t *>(gate),
                          static_cast<const uint8_t *>(up), static_cast<const uint8_t *>(down));
}

// raw rows of `count` experts into the gate | up | down slots at dst, then the packed / tile-major copies of experts first .. first + count - 1
static int stage_and_pack(Moe *m, uint32_t layer, uint32_t first, uint32_t count, uint8_t *dst, const uint8_t *gate, const uint8_t *up, const uint8_t *down) {
    // 2-D copies place the tightly packed source matrices into the gate | up | down slots
    HIP_OK(hipMemcpy2D(dst, m->expert_stride, gate, m->gate_bytes, m->gate_bytes, count, hipMemcpyDefault), "expert gate upload");
    HIP_OK(hipMemcpy2D(dst + m->gate_bytes, m->expert_stride, up, m->gate_bytes, m->gate_bytes, count, hipMemcpyDefault), "expert up upload");
    HIP_OK(hipMemcpy2D(dst + 2u * m->gate_bytes, m->expert_stride, down, m->down_bytes, m->down_bytes, count, hipMemcpyDefault), "expert down upload");
    if (m->packed_gu()) {
        const redhip_moe_config &c = m->cfg;
        uint8_t *pk = m->layers[layer].packed + (uint64_t)first * m->packed_stride;
        HIP_OK(launch_repack_gateup(m->gu_type, dst, m->expert_stride, count, c.ffn, c.hidden, pk, m->packed_stride, nullptr), "expert gate repack");
        HIP_OK(launch_repack_gateup(m->gu_type, dst + m->gate_bytes, m->expert_stride, count, c.ffn, c.hidden, pk + m->pk_gate_bytes, m->packed_stride, nullptr), "expert up repack");
        // row-major packed down matrices: beside gate | up where the layout keeps them, else in the staging buffer (source of the tiles only)
        const uint8_t *pk_down = nullptr;
        uint64_t pk_down_stride = 0;
        if (m->fused) {
            if (m->rowmajor_down()) {
                HIP_OK(launch_repack_iq2xxs(dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn, false, pk + 2u * m->gate_bytes, m->packed_stride, nullptr), "expert down repack");
                pk_down = pk + 2u * m->gate_bytes;
                pk_down_stride = m->packed_stride;
            } else if (m->layers[layer].tiled) {
                if (!m->stage_down || count > Moe::kStageExperts) { moe_err("down staging buffer missing"); return 0; }
                HIP_OK(launch_repack_iq2xxs(dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn, false, m->stage_down, m->down_cm_stride(), nullptr), "expert down repack");
                pk_down = m->stage_down;
                pk_down_stride = m->down_cm_stride();
            }
            HIP_OK(launch_repack_iq2xxs(dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn, true,
                                        m->layers[layer].down_cm + (uint64_t)first * m->down_cm_stride(), m->down_cm_stride(), nullptr), "expert down column slices");
        }
        if (m->layers[layer].tiled) {      // (the tile-major copy keeps the gate | up | down slots of the raw layout)
            const uint64_t tstride = m->tiled_stride();
            uint8_t *tl = m->layers[layer].tiled + (uint64_t)first * tstride;
            const bool gu_sc = m->gu_type == T_IQ2_XS;          // its streams carry a scale byte per group
            HIP_OK(launch_tile_packed(pk, m->packed_stride, count, c.ffn, c.hidden, tl, tstride, nullptr, gu_sc), "expert gate tiling");
            HIP_OK(launch_tile_packed(pk + m->pk_gate_bytes, m->packed_stride, count, c.ffn, c.hidden, tl + m->pk_gate_bytes, tstride, nullptr, gu_sc), "expert up tiling");
            if (m->fused)
                HIP_OK(launch_tile_packed(pk_down, pk_down_stride, count, c.hidden, c.ffn, tl + 2u * m->gate_bytes, tstride, nullptr), "expert down tiling");
        }
        if (m->layers[layer].words_down) {
            uint8_t *wd = m->layers[layer].words_down + (uint64_t)first * m->words_down_stride();
            if (m->dn_type == T_IQ3_S) HIP_OK(launch_repack_iq3s_words(dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn, wd, m->words_down_stride(), nullptr), "expert down words");
            else HIP_OK(launch_repack_gateup(m->dn_type, dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn, wd, m->words_down_stride(), nullptr), "expert down streams");
        }
        if (m->sliced_words())
            HIP_OK(launch_repack_iq3s_words(dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn, m->layers[layer].down_cm + (uint64_t)first * m->down_cm_stride(),
                                            m->down_cm_stride(), nullptr, true), "expert down column slices");
        if (m->sliced_streams())
            HIP_OK(launch_repack_gateup(m->dn_type, dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn,
                                        m->layers[layer].down_cm + (uint64_t)first * m->down_cm_stride(), m->down_cm_stride(), nullptr, true), "expert down column slices");
        if (m->layers[layer].tiled_down && m->dn_type == T_IQ3_S)
            HIP_OK(launch_tile_iq3s(dst + 2u * m->gate_bytes, m->expert_stride, count, c.hidden, c.ffn,
                                    m->layers[layer].tiled_down + (uint64_t)first * m->tiled_down_stride(), m->tiled_down_stride(), nullptr), "expert down tiling");
        if (m->layers[layer].tiled_down && m->dn_type != T_IQ3_S) {      // IQ2_XS / IQ1_M: the tile-major copy of the row-major streams written above
            if (!m->layers[layer].words_down) { moe_err("internal: no row-major down streams to tile"); return 0; }
            HIP_OK(launch_tile_packed(m->layers[layer].words_down + (uint64_t)first * m->words_down_stride(), m->words_down_stride(), count, c.hidden, c.ffn,
                                      m->layers[layer].tiled_down + (uint64_t)first * m->words_down_stride(), m->words_down_stride(), nullptr, m->dn_type == T_IQ2_XS),
                   "expert down tiling");
        }
        HIP_OK(hipStreamSynchronize(nullptr), "expert repack");
    }
    return 1;
}

int redhip_moe_route(redhip_moe_t h, uint32_t layer, const float *x_dev, uint32_t ntok, uint32_t *ids_dev, float *weights_dev,
                     float *logits_dev, void *stream) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    const redhip_moe_config &c = m->cfg;
    if (!x_dev || !ntok || ntok > c.max_tokens) { moe_err("invalid token count %u (max %u)", ntok, c.max_tokens); return 0; }
    hipStream_t s = static_cast<hipStream_t>(stream);
    float *lg = logits_dev ? logits_dev : m->logits;
    if (m->fast_route()) {
        prof_set_stage(ST_ROUTER_GEMV);
        // a Q6_K shared expert of a mixed layout rides along: its gate / up products land in m->act (otherwise unused on this path)
        const float *router_f32 = c.router_type == T_F32 ? reinterpret_cast<const float *>(m->layers[layer].router) : m->layers[layer].dense_router;
        // one token or a small batch on a mixed layout: the router and the shared expert's gate | up rows as one f32 GEMV over their f32 copies
        // (4.5 times the bytes of the Q6_K rows, none of their decode arithmetic)
        const uint32_t nv = c.hidden / 256u;
        const bool dense_small = m->mixed && router_f32 && m->layers[layer].dense_gu && (ntok == 1u || m->small_batch_mixed(ntok)) && c.top_k >= 2u &&
                                 (nv == 2u || nv == 4u || nv == 8u || nv == 16u);
        m->shared_gu_ready = dense_small ||
                             (m->mixed && m->sh_gu_type == T_Q6_K && c.router_type == T_Q6_K && (ntok == 1u || m->small_batch_mixed(ntok)) && c.top_k >= 2u);
        const bool dense_multi = !dense_small && m->mixed && ntok > 8u && m->small_batch(ntok, true) && router_f32 && m->layers[layer].dense_gu;
        if (dense_multi) {
            // 9..32 tokens on a mixed layout whose batches run as slices: the launch of the small batches once per sixteen tokens, each
            // on its own rows of the activations, logits, fp16 halves and shared products (a block step: of the branch and the normalised rows too)
            BlockContext &bc = block_context();
            const BlockContext saved = bc;
            const uint32_t per = (size_t)16u * c.hidden * 4u <= 128u * 1024u ? 16u : 8u;      // tokens whose activations fit the launch's LDS
            for (uint32_t t0 = 0; t0 < ntok; t0 += per) {
                const uint32_t n = ntok - t0 < per ? ntok - t0 : per;
                const size_t row = (size_t)t0 * c.hidden;
                if (saved.branch) { bc.branch = saved.branch + row; bc.xn_out = saved.xn_out + row; }
                const hipError_t e = launch_router_gemv(T_F32, router_f32, x_dev + row, m->layers[layer].gate_inp, n, c.hidden, c.n_expert,
                                                        m->logits + (size_t)t0 * (c.n_expert + 1u), static_cast<uint8_t *>(m->xh) + 2u * row,
                                                        static_cast<uint8_t *>(m->xl) + 2u * row, m->xexp + t0, nullptr, m->act + (size_t)t0 * 2u * c.ffn, c.ffn, s,
                                                        m->layers[layer].dense_gu);
                if (e != hipSuccess) { bc = saved; HIP_OK(e, "router launch"); }
            }
            bc = saved;
            m->shared_gu_ready = true;
        } else if (m->tiled_router(ntok))
            HIP_OK(launch_router_f32_tiles(router_f32, m->layers[layer].gate_inp, x_dev, ntok, c.hidden,
                                           c.n_expert, m->logits, m->xh, m->xl, m->xexp, s), "router tile launch");
        else if (dense_small)
            HIP_OK(launch_router_gemv(T_F32, router_f32, x_dev, m->layers[layer].gate_inp, ntok, c.hidden, c.n_expert, m->logits, m->xh, m->xl, m->xexp,
                                      nullptr, m->act, c.ffn, s, m->layers[layer].dense_gu), "router launch");
        else if (m->mixed && c.router_type != T_F32 && router_f32 && ntok > 8u && (nv == 2u || nv == 4u || nv == 8u || nv == 16u))
            // a small chunk on a layout with a quantised router: the f32 copy of its rows, one token per grid layer (no shared rows: the
            // shared expert of a chunk runs as dense products on the second stream)
            HIP_OK(launch_router_gemv(T_F32, router_f32, x_dev, m->layers[layer].gate_inp, ntok, c.hidden, c.n_expert, m->logits, m->xh, m->xl, m->xexp,
                                      nullptr, nullptr, c.ffn, s), "router launch");
        else
            HIP_OK(launch_router_gemv(c.router_type, m->layers[layer].router, x_dev, m->layers[layer].gate_inp, ntok, c.hidden, c.n_expert,
                                      m->logits, m->xh, m->xl, m->xexp, m->shared_gu_ready ? m->layers[layer].shared : nullptr, m->act, c.ffn, s),
                   "router launch");
        if (!m->skip_select) {
            prof_set_stage(ST_ROUTE_SELECT);
            HIP_OK(launch_select(m->logits, ntok, c.n_expert, c.top_k, ids_dev ? ids_dev : m->ids, weights_dev ? weights_dev : m->weights,
                                 m->scalar, nullptr, s), "selection launch");
        }
        prof_set_stage(ST_OTHER);
        if (logits_dev) HIP_OK(hipMemcpy2DAsync(logits_dev, 4u * (size_t)c.n_expert, m->logits, 4u * (size_t)(c.n_expert + 1u), 4u * (size_t)c.n_expert,
                                                ntok, hipMemcpyDeviceToDevice, s), "logits copy");
        return 1;
    }
    prof_set_stage(ST_ROUTER_GEMV);
    for (uint32_t t = 0; t < ntok; ++t)
        HIP_OK(launch_gemv_rows(c.router_type, m->layers[layer].router, c.hidden, 0u, c.n_expert, x_dev + (size_t)t * c.hidden,
                                lg + (size_t)t * c.n_expert, s), "router GEMV launch");
    prof_set_stage(ST_ROUTE_SELECT);
    HIP_OK(launch_route_select(lg, ntok, c.n_expert, c.top_k, ids_dev ? ids_dev : m->ids, weights_dev ? weights_dev : m->weights, nullptr,
                               m->layers[layer].gate_inp, x_dev, c.hidden, m->scalar, s), "router selection launch");
    prof_set_stage(ST_OTHER);
    return 1;
}

int redhip_moe_experts(redhip_moe_t h, uint32_t layer, const float *x_dev, uint32_t ntok, const uint32_t *ids_dev,
                       const float *weights_dev, float *out_dev, void *stream) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    if (!x_dev || !ids_dev || !weights_dev || !out_dev || !ntok || ntok > m->cfg.max_tokens) { moe_err("invalid expert execution arguments"); return 0; }
    hipStream_t s = static_cast<hipStream_t>(stream);
    m->shared_gu_ready = false;
    struct GuardScope {          // the caller's ids are clamped and reported by every kernel that reads them during this call
        GuardScope(uint32_t n, uint32_t *st) { route_guard() = RouteGuard{n, st}; }
        ~GuardScope() { route_guard() = RouteGuard{}; }
    } guard_scope(m->cfg.n_expert, m->status);
    if (m->packed_path(ntok) || m->small_batch_mixed(ntok) || m->mixed_chunk(ntok) || m->stream_chunk(ntok)) {
        const Layer &L = m->layers[layer];
        const uint32_t nv = m->cfg.hidden / 256u;
        // batches whose pairs are grouped by expert next: the pair sort rides in the same launch as one more workgroup
        // (with the routing given, grouping pays from two tokens on: the pair sort costs no launch of its own)
        const bool to_group = m->small_batch(ntok) || m->grouped_mixed(ntok, 2u);
        const GroupJob job{ids_dev, weights_dev, ntok, m->cfg.top_k, m->cfg.n_expert, m->uid, m->expert_start, m->pair_token, m->pair_weight, m->tok_pair, m->n_unique, m->status,
                           m->small_batch(ntok) ? m->pass_list : nullptr, m->small_batch(ntok) ? m->n_pass : nullptr};
        bool grouped = false;
        const bool mixed_mid = m->mixed_slices && ntok > 8u && ntok <= Moe::kSmallMaxGiven && m->small_batch(ntok, true) && L.dense_gu;
        if (mixed_mid) {
            // 9..24 tokens on a mixed layout whose batches run as slices: the shared expert's products, the fp16 halves and the scalar gates
            // from the launch of the small batches, once per sixteen tokens; then one launch sorts the pairs with their pass list
            prof_set_stage(ST_SHARED_GATEUP);
            const uint32_t per = (size_t)16u * m->cfg.hidden * 4u <= 128u * 1024u ? 16u : 8u;      // tokens whose activations fit the launch's LDS
            for (uint32_t t0 = 0; t0 < ntok; t0 += per) {
                const uint32_t n = ntok - t0 < per ? ntok - t0 : per;
                const size_t row = (size_t)t0 * m->cfg.hidden;
                HIP_OK(launch_router_gemv(T_F32, L.dense_gu, x_dev + row, L.gate_inp, n, m->cfg.hidden, 0u, m->logits + t0, static_cast<uint8_t *>(m->xh) + 2u * row,
                                          static_cast<uint8_t *>(m->xl) + 2u * row, m->xexp + t0, nullptr, m->act + (size_t)t0 * 2u * m->cfg.ffn, m->cfg.ffn, s, L.dense_gu,
                                          m->scalar + t0), "shared gate/up launch");
            }
            m->shared_gu_ready = true;
            const GroupJob big{ids_dev, weights_dev, ntok, m->cfg.top_k, m->cfg.n_expert, m->uid, m->expert_start, m->pair_token, m->pair_weight, m->tok_pair, m->n_unique,
                               m->status, m->pass_list, m->n_pass};
            prof_set_stage(ST_GROUP);
            HIP_OK(launch_group_small(big, s), "pair sort launch");
            grouped = true;
        } else if (m->mixed && m->packed_gu() && (ntok == 1u || m->small_batch_mixed(ntok)) && L.dense_gu && (nv == 2u || nv == 4u || nv == 8u || nv == 16u)) {
            // one token or a small batch on a mixed layout: the kernels take the shared expert's gate | up products as an input: one f32
            // GEMV over its f32 copy (no router rows), which also leaves the fp16 halves of x and the shared expert's scalar gate
            prof_set_stage(ST_SHARED_GATEUP);
            HIP_OK(launch_router_gemv(T_F32, L.dense_gu, x_dev, L.gate_inp, ntok, m->cfg.hidden, 0u, m->logits, m->xh, m->xl, m->xexp, nullptr, m->act,
                                      m->cfg.ffn, s, L.dense_gu, m->scalar, to_group ? &job : nullptr, &grouped), "shared gate/up launch");
            m->shared_gu_ready = true;
        } else {
            prof_set_stage(ST_OTHER);
            HIP_OK(launch_prep(x_dev, L.gate_inp, ntok, m->cfg.hidden, m->xh, m->xl, m->xexp, m->scalar, s, to_group ? &job : nullptr, &grouped), "prep launch");
        }
        if (m->fused && !grouped && !m->small_batch(ntok) && m->small_batch(ntok, true) && ntok <= Moe::kSmallMaxGiven) {
            // 17..24 tokens on an all-IQ2_XXS layer: more pairs than the side job above sorts; one more launch sorts them with their pass list.
            // (The slices cost a pass per two pairs of an expert, the tile kernels a decode per distinct expert: with 32 hot experts the
            // slices took 58.5 / 74.2 / 93.2 us at 17 / 24 / 32 tokens against 67.9 / 79.2 / 84.5 us on the tiles.)
            const GroupJob big{ids_dev, weights_dev, ntok, m->cfg.top_k, m->cfg.n_expert, m->uid, m->expert_start, m->pair_token, m->pair_weight, m->tok_pair, m->n_unique,
                               m->status, m->pass_list, m->n_pass};
            prof_set_stage(ST_GROUP);
            HIP_OK(launch_group_small(big, s), "pair sort launch");
            grouped = true;
        }
        const int ok = experts_enqueue(m, layer, x_dev, ntok, ids_dev, weights_dev, out_dev, s, false, grouped);
        m->shared_gu_ready = false;
        return ok;
    }
    scalar_gate_kernel<<<ntok, 256, 0, s>>>(m->layers[layer].gate_inp, x_dev, m->cfg.hidden, m->scalar);
    HIP_OK(hipGetLastError(), "scalar gate launch");
    return experts_enqueue(m, layer, x_dev, ntok, ids_dev, weights_dev, out_dev, s);
}

int redhip_moe_forward(redhip_moe_t h, uint32_t layer, const float *x_dev, uint32_t ntok, float *out_dev, void *stream) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    if (!x_dev || !out_dev) { moe_err("null activation pointer"); return 0; }
    if (m->sliced(ntok) && ntok <= m->cfg.max_tokens) {
        int ok = 1;
        for (uint32_t t0 = 0; t0 < ntok && ok; t0 += Moe::kSlice) {
            const uint32_t n = ntok - t0 < Moe::kSlice ? ntok - t0 : Moe::kSlice;
            m->shift_route_outputs(t0);
            ok = redhip_moe_forward(h, layer, x_dev + (size_t)t0 * m->cfg.hidden, n, out_dev + (size_t)t0 * m->cfg.hidden, stream);
            m->shift_route_outputs(-(int64_t)t0);
        }
        return ok;
    }
    const bool group_in_select = m->slices_after_router(ntok) || m->grouped_mixed(ntok);
    const bool select_in_gateup = m->packed_gu() && (ntok == 1u || m->small_batch_mixed(ntok)) && !group_in_select;
    m->skip_select = select_in_gateup || group_in_select;      // small batches: the batched gate/up kernel selects and sorts the pairs itself
    const int routed = redhip_moe_route(h, layer, x_dev, ntok, nullptr, nullptr, nullptr, stream);
    m->skip_select = false;
    if (!routed) return 0;
    if (m->slices_after_router(ntok)) return select_group_slices(m, layer, x_dev, ntok, out_dev, static_cast<hipStream_t>(stream));
    return experts_enqueue(m, layer, x_dev, ntok, m->ids, m->weights, out_dev, static_cast<hipStream_t>(stream), select_in_gateup || group_in_select, group_in_select);
}

int redhip_moe_forward_block(redhip_moe_t h, uint32_t layer, const float *x_dev, const float *branch_dev, const float *post_norm_dev, float eps,
                             uint32_t ntok, float *x_out_dev, void *stream) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    if (!x_dev || !branch_dev || !post_norm_dev || !x_out_dev || !ntok || ntok > m->cfg.max_tokens) { moe_err("invalid block step arguments"); return 0; }
    const redhip_moe_config &c = m->cfg;
    if (m->sliced(ntok)) {
        int ok = 1;
        for (uint32_t t0 = 0; t0 < ntok && ok; t0 += Moe::kSlice) {
            const uint32_t n = ntok - t0 < Moe::kSlice ? ntok - t0 : Moe::kSlice;
            const size_t off = (size_t)t0 * c.hidden;
            m->shift_route_outputs(t0);
            float *xn = m->xn;
            m->xn += off;                                // the normalised rows of the slice at their place in the chunk too
            ok = redhip_moe_forward_block(h, layer, x_dev + off, branch_dev + off, post_norm_dev, eps, n, x_out_dev + off, stream);
            m->xn = xn;
            m->shift_route_outputs(-(int64_t)t0);
        }
        return ok;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    BlockContext &bc = block_context();
    bc = BlockContext{};
    // the per-token router kernels of the packed paths normalise on the fly; everything else gets a kernel of its own
    const bool in_router = m->fast_route() && !m->tiled_router(ntok);
    int ok = 1;
    if (!in_router) {
        prof_set_stage(ST_OTHER);
        resid_rms_kernel<<<ntok, 256, 0, s>>>(x_dev, branch_dev, post_norm_dev, eps, c.hidden, m->xn);
        if (hipGetLastError() != hipSuccess) { moe_err("residual + norm launch failed"); ok = 0; }
    }
    if (ok) {
        const bool group_in_select = m->slices_after_router(ntok) || m->grouped_mixed(ntok);
        const bool select_in_gateup = m->packed_gu() && (ntok == 1u || m->small_batch_mixed(ntok)) && !group_in_select;
        m->skip_select = select_in_gateup || group_in_select;
        if (in_router) { bc.branch = branch_dev; bc.norm_w = post_norm_dev; bc.eps = eps; bc.xn_out = m->xn; }
        ok = redhip_moe_route(h, layer, in_router ? x_dev : m->xn, ntok, nullptr, nullptr, nullptr, stream);
        bc.branch = bc.norm_w = nullptr;
        bc.xn_out = nullptr;
        m->skip_select = false;
            if (ok) {
            bc.resid_a = x_dev;                              // the path's last kernel adds x + branch to its output
            bc.resid_b = branch_dev;
            ok = m->slices_after_router(ntok) ? select_group_slices(m, layer, m->xn, ntok, x_out_dev, s)
                                      : experts_enqueue(m, layer, m->xn, ntok, m->ids, m->weights, x_out_dev, s, select_in_gateup || group_in_select, group_in_select);
        }
    }
    bc = BlockContext{};
    return ok;
}

int redhip_moe_last_route(redhip_moe_t h, uint32_t ntok, uint32_t *ids, float *weights, float *logits, void *stream) {
    Moe *m = moe_of(h);
    if (!m || !ntok || ntok > m->cfg.max_tokens) { moe_err("invalid last-route request"); return 0; }
    HIP_OK(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "stream synchronise");
    const redhip_moe_config &c = m->cfg;
    uint32_t status = 0u;
    HIP_OK(hipMemcpy(&status, m->status, 4u, hipMemcpyDeviceToHost), "status download");
    if (status) {
        HIP_OK(hipMemset(m->status, 0, 4u), "status reset");
        moe_err("routing given to redhip_moe_experts / redhip_moe_group broke its contract:%s%s (ids were clamped; the outputs of those calls are not meaningful)",
                (status & 1u) ? " an expert id was >= n_expert" : "", (status & 2u) ? " a token named an expert twice" : "");
        return 0;
    }
    if (ids) HIP_OK(hipMemcpy(ids, m->ids, (size_t)ntok * c.top_k * 4u, hipMemcpyDeviceToHost), "ids download");
    if (weights) HIP_OK(hipMemcpy(weights, m->weights, (size_t)ntok * c.top_k * 4u, hipMemcpyDeviceToHost), "weights download");
    if (logits) {
        const size_t pitch = 4u * (size_t)(c.n_expert + (m->fast_route() ? 1u : 0u));
        HIP_OK(hipMemcpy2D(logits, 4u * (size_t)c.n_expert, m->logits, pitch, 4u * (size_t)c.n_expert, ntok, hipMemcpyDeviceToHost), "logits download");
    }
    return 1;
}

int redhip_moe_group(redhip_moe_t h, const uint32_t *ids_dev, const float *weights_dev, uint32_t ntok, uint32_t *uid_dev,
                     uint32_t *expert_start_dev, uint32_t *pair_token_dev, float *pair_weight_dev, uint32_t *tok_pair_dev,
                     uint32_t *n_unique_dev, void *stream) {
    Moe *m = moe_of(h);
    if (!m) { moe_err("null MoE handle"); return 0; }
    if (!ids_dev || !weights_dev || !uid_dev || !expert_start_dev || !pair_token_dev || !pair_weight_dev || !tok_pair_dev || !n_unique_dev || !ntok) {
        moe_err("invalid grouping arguments");
        return 0;
    }
    prof_set_stage(ST_GROUP);
    route_guard() = RouteGuard{m->cfg.n_expert, m->status};
    const hipError_t ge = launch_group_pairs(ids_dev, weights_dev, ntok, m->cfg.top_k, m->cfg.n_expert, uid_dev, expert_start_dev, pair_token_dev,
                                             pair_weight_dev, tok_pair_dev, n_unique_dev, static_cast<hipStream_t>(stream), nullptr,
                                             ntok <= m->cfg.max_tokens ? m->group_scratch_ptr() : nullptr);
    route_guard() = RouteGuard{};
    HIP_OK(ge, "grouping launch");
    return 1;
}

int redhip_set_codebooks(const int8_t *iq2_xs_grid, uint32_t iq2_xs_count, const int8_t *iq1_m_grid, uint32_t iq1_m_count) {
    if ((iq2_xs_grid && iq2_xs_count != 512u * 8u) || (iq1_m_grid && iq1_m_count != 2048u * 8u)) {
        moe_err("codebook size mismatch: IQ2_XS takes 4096 values, IQ1_M 16384");
        return 0;
    }
    const hipError_t e = set_caller_grids(iq2_xs_grid, iq1_m_grid);
    if (e == hipErrorContextAlreadyInUse) { moe_err("%s", kCodebookConflict); return 0; }
    HIP_OK(e, "codebook upload");
    return 1;
}

int redhip_dequant_rows(uint32_t ggml_type, const void *rows_dev, uint32_t nrows, uint32_t ncols, float *out_dev, void *stream) {
    if (!rows_dev || !out_dev) { moe_err("null dequant pointer"); return 0; }
    HIP_OK(launch_dequant_rows(ggml_type, rows_dev, nrows, ncols, out_dev, static_cast<hipStream_t>(stream)), "dequant launch");
    return 1;
}

int redhip_moe_dequant_resident(redhip_moe_t h, uint32_t layer, uint32_t expert, uint32_t which, float *out_dev, void *stream) {
    Moe *m = moe_of(h);
    if (!check_layer(m, layer)) return 0;
    const redhip_moe_config &c = m->cfg;
    if (!out_dev || which > 4u || (which != 3u && expert > c.n_expert)) { moe_err("invalid resident matrix request"); return 0; }
    const Layer &L = m->layers[layer];
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (which == 3u) { HIP_OK(launch_dequant_rows(c.router_type, L.router, c.n_expert, c.hidden, out_dev, s), "router dequant"); return 1; }
    const bool sh = expert == c.n_expert;
    if (which == 4u) {                                      // the column-sliced copy of a down matrix
        if (m->sliced_words() && !sh) {
            HIP_OK(launch_dequant_iq3s_words(L.down_cm + (uint64_t)expert * m->down_cm_stride(), c.hidden, c.ffn, out_dev, s, true), "column-sliced down dequant");
            return 1;
        }
        if (m->sliced_streams() && !sh) {
            HIP_OK(launch_dequant_packed(m->dn_type, L.down_cm + (uint64_t)expert * m->down_cm_stride(), c.hidden, c.ffn, m->dn_grid, out_dev, s, true), "column-sliced down dequant");
            return 1;
        }
        if (!m->fused) { moe_err("this layout keeps no column-sliced copy of that down matrix"); return 0; }
        HIP_OK(launch_dequant_packed_iq2xxs(sh ? L.shared_down_cm : L.down_cm + (uint64_t)expert * m->down_cm_stride(), c.hidden, c.ffn, true, out_dev, s), "column-sliced down dequant");
        return 1;
    }
    if (m->fused || (m->mixed && which < 2u && (!sh || L.shared_packed))) {        // the layout the MFMA kernels read
        const uint8_t *pk = sh ? L.shared_packed : L.packed + (uint64_t)expert * m->packed_stride;
        const uint64_t gbytes = m->pk_gate_bytes;
        if (which < 2u) HIP_OK(launch_dequant_packed(m->gu_type, pk + which * gbytes, c.ffn, c.hidden, m->gu_grid, out_dev, s), "packed gate/up dequant");
        else if (sh || m->rowmajor_down()) HIP_OK(launch_dequant_packed_iq2xxs(pk + 2u * gbytes, c.hidden, c.ffn, false, out_dev, s), "packed down dequant");
        else HIP_OK(launch_dequant_packed_iq2xxs(L.down_cm + (uint64_t)expert * m->down_cm_stride(), c.hidden, c.ffn, true, out_dev, s), "column-sliced down dequant");
        return 1;
    }
    if (which == 2u && !sh && m->sliced_words()) {
        HIP_OK(launch_dequant_iq3s_words(L.down_cm + (uint64_t)expert * m->down_cm_stride(), c.hidden, c.ffn, out_dev, s, true), "column-sliced down dequant");
        return 1;
    }
    if (which == 2u && !sh && L.words_down) {       // the copy the MFMA down kernels read
        const uint8_t *wd = L.words_down + (uint64_t)expert * m->words_down_stride();
        if (m->dn_type == T_IQ3_S) HIP_OK(launch_dequant_iq3s_words(wd, c.hidden, c.ffn, out_dev, s), "word-packed down dequant");
        else HIP_OK(launch_dequant_packed(m->dn_type, wd, c.hidden, c.ffn, m->dn_grid, out_dev, s), "stream-packed down dequant");
        return 1;
    }
    if (!sh && !raw_rows(m, layer)) return 0;
    const uint8_t *base = sh ? L.shared : L.experts + (uint64_t)expert * m->expert_stride;
    const uint64_t gb = sh ? m->sh_gate_bytes : m->gate_bytes;
    const uint32_t gu = sh ? m->sh_gu_type : m->gu_type, dn = sh ? m->sh_dn_type : m->dn_type;
    if (which == 0u) HIP_OK(launch_dequant_rows(gu, base, c.ffn, c.hidden, out_dev, s), "gate dequant");
    else if (which == 1u) HIP_OK(launch_dequant_rows(gu, base + gb, c.ffn, c.hidden, out_dev, s), "up dequant");
    else HIP_OK(launch_dequant_rows(dn, base + 2u * gb, c.hidden, c.ffn, out_dev, s), "down dequant");
    return 1;
}

int redhip_gemv_rows(uint32_t ggml_type, const void *matrix_dev, uint32_t ncols, uint32_t row_start, uint32_t row_count,
                     const float *x_dev, float *out_dev, void *stream) {
    if (!matrix_dev || !x_dev || !out_dev) { moe_err("null GEMV pointer"); return 0; }
    HIP_OK(launch_gemv_rows(ggml_type, matrix_dev, ncols, row_start, row_count, x_dev, out_dev, static_cast<hipStream_t>(stream)), "GEMV launch");
    return 1;
}

}  // extern "C"
