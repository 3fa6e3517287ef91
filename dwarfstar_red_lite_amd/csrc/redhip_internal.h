// Internal interface between the C-ABI front ends and the gfx950 kernels of libredmetal_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>

#include <mutex>

namespace redhip {

std::mutex &caller_grid_mutex();      // serialises uploads of the caller-supplied codebooks (and one-shot launches that must see their own)

enum : uint32_t { T_F32 = 0u, T_Q6_K = 14u, T_IQ2_XXS = 16u, T_IQ2_XS = 17u, T_IQ3_S = 21u, T_IQ1_M = 29u };

// bytes per 256 weights; 0 for a type this library does not decode. IQ2_XS and IQ1_M (the reference's current routed
// formats, codebooks supplied by the caller) are decoded by the pool and one-shot GEMV surfaces only.
inline uint32_t block_bytes(uint32_t t) { return t == T_Q6_K ? 210u : t == T_IQ2_XXS ? 66u : t == T_IQ3_S ? 110u : 0u; }
inline uint32_t pool_block_bytes(uint32_t t) { return t == T_IQ2_XS ? 74u : t == T_IQ1_M ? 56u : block_bytes(t); }
inline uint64_t pool_row_bytes(uint32_t t, uint32_t ncols) {
    if (t == T_F32) return 4ull * ncols;
    const uint32_t b = pool_block_bytes(t);
    return (b && ncols && ncols % 256u == 0u) ? (uint64_t)(ncols / 256u) * b : 0ull;
}
inline bool pool_quant_supported(uint32_t t) { return pool_block_bytes(t) != 0u; }
// device copies of the caller's IQ2_XS (512 x 8) / IQ1_M (2048 x 8) int8 codebooks; either may be null (left as is).
// One pair per process. `bind_owner` (a pool, a resident-layer handle) binds itself to the content it uploads; while anybody is bound an
// upload of different content returns hipErrorContextAlreadyInUse (report it with kCodebookConflict) instead of changing what the bound
// users decode through; the same content again is free. forget_caller_grids unbinds.
hipError_t set_caller_grids(const int8_t *iq2_xs, const int8_t *iq1_m, const void *bind_owner = nullptr);
hipError_t set_caller_grids_locked(const int8_t *iq2_xs, const int8_t *iq1_m, const void *bind_owner = nullptr);      // caller holds caller_grid_mutex()
bool caller_grids_bound(const void *owner);
void forget_caller_grids(const void *owner);
constexpr const char *kCodebookConflict = "IQ2_XS / IQ1_M codebooks differ from the ones this process holds while pools or resident layers that decode through them are alive";
const int8_t *caller_grid_device(uint32_t type);      // device address of the process's codebook of IQ2_XS / IQ1_M, nullptr for other types
bool caller_grid_present(uint32_t type);       // true for the formats that carry their own tables
inline uint64_t row_bytes(uint32_t t, uint32_t ncols) {
    if (!ncols) return 0;
    if (t == T_F32) return 4ull * ncols;
    const uint32_t b = block_bytes(t);
    return (b && ncols % 256u == 0u) ? (uint64_t)(ncols / 256u) * b : 0ull;
}
inline bool quant_supported(uint32_t t) { return block_bytes(t) != 0u; }
// the reference's two-type word: gate/up in bits 0-7, down in bits 8-15 when it differs
inline uint32_t word_gate_up(uint32_t w) { return w & 255u; }
inline uint32_t word_down(uint32_t w) { return ((w >> 8) & 255u) ? ((w >> 8) & 255u) : (w & 255u); }

// ---- per-stage kernel timing (off unless redhip_profile_begin was called) ----
// When on, every kernel launch carries a start and a stop event whose timestamps are the dispatch's own begin
// and end, so a stage's time is kernel execution only, not launch latency.
enum Stage : uint32_t {
    ST_OTHER = 0, ST_ROUTER_GEMV, ST_ROUTE_SELECT, ST_GROUP, ST_GATEUP, ST_SHARED_GATEUP, ST_DOWN_COMBINE,
    ST_FUSED_EXPERTS, ST_BATCH_GATEUP, ST_BATCH_DOWN, ST_BATCH_COMBINE, ST_PREFILL_GATEUP, ST_PREFILL_DOWN, ST_SLICE_SUM, ST_COUNT
};
void prof_set_stage(uint32_t stage);                       // label of the launches that follow (calling thread)

// The step around the layer (native/redlite_native_engine_cpu.c:418-427): the layer's input is the RMS-norm of x + branch,
// and x + branch is added to its output. Both are context of the calling thread, picked up by the launchers below:
// the router launchers normalise on the fly and write the normalised activations to xn_out, the launchers of a path's
// last kernel add resid_a[i] + resid_b[i] to out[i]. All null outside redhip_moe_forward_block.
struct BlockContext {
    const float *branch = nullptr, *norm_w = nullptr;      // router side: x := (x + branch) * rsqrt(mean((x + branch)^2) + eps) * norm_w
    float eps = 0.0f;
    float *xn_out = nullptr;
    const float *resid_a = nullptr, *resid_b = nullptr;   // output side
};
BlockContext &block_context();

// Routing that a caller hands in (redhip_moe_experts, redhip_moe_group) is untrusted: every kernel that turns an expert id into an
// address clamps it to id_limit - 1 first and, when it had to, sets bit 0 of *status; the pair sort sets bit 1 when a token names an
// expert twice (its bitmap ranks assume distinct ids per token). Context of the calling thread, picked up by the launchers; the default
// clamps nothing and reports nowhere (ids the library selected itself).
struct RouteGuard {
    uint32_t id_limit = 0xffffffffu;      // n_expert
    uint32_t *status = nullptr;           // device word
};
RouteGuard &route_guard();
#if defined(__HIPCC__)
__device__ __forceinline__ uint32_t guarded_id(uint32_t id, uint32_t id_limit, uint32_t *status) {
    if (id < id_limit) return id;
    if (status) atomicOr(status, 1u);
    return id_limit - 1u;
}
#endif
void prof_events(hipEvent_t *start, hipEvent_t *stop);     // both nullptr when profiling is off

#define REDHIP_LAUNCH(kern, grid, block, lds, stream, ...)                                         \
    do {                                                                                           \
        hipEvent_t ev_a_ = nullptr, ev_b_ = nullptr;                                               \
        ::redhip::prof_events(&ev_a_, &ev_b_);                                                     \
        hipExtLaunchKernelGGL(kern, grid, block, lds, stream, ev_a_, ev_b_, 0u, __VA_ARGS__);      \
    } while (0)

// ---- launchers (enqueue only; return hipSuccess or the launch error) ----

hipError_t launch_dequant_rows(uint32_t type, const void *rows, uint32_t nrows, uint32_t ncols, float *out, hipStream_t s);

// out[r] = W[row_start + r] . x for r < row_count; raw GGUF rows
hipError_t launch_gemv_rows(uint32_t type, const void *w, uint32_t ncols, uint32_t row_start, uint32_t row_count,
                            const float *x, float *out, hipStream_t s);

// act[i] = SiLU(gate[i]) * up[i]
hipError_t launch_silu_mul(const float *gate, const float *up, float *act, uint32_t n, hipStream_t s);

// per token: softmax over n_expert logits, top_k by probability (ties to lower index), renormalised weights;
// optional probs [ntok][n_expert]; optional shared scalar gate sigmoid(gate_inp . x_t) -> scalar[t]
hipError_t launch_route_select(const float *logits, uint32_t ntok, uint32_t n_expert, uint32_t top_k,
                               uint32_t *ids, float *weights, float *probs,
                               const float *gate_inp, const float *x, uint32_t hidden, float *scalar, hipStream_t s);

struct ExpertSet {               // where the experts of one layer live (raw GGUF layout, gate|up|down per expert)
    const uint8_t *base;         // expert e starts at base + e * stride
    uint64_t stride;
    uint64_t gate_bytes, up_bytes;
    uint32_t gate_up_type, down_type;
    const uint64_t *table = nullptr;   // device array of expert base addresses (a slot table), or nullptr. When set, slot / group i
                                       // reads its expert at table[i]; base, stride and the ids / uid arrays are not used
};

// act[slot][r] = SiLU(gate_e[r] . x) * (up_e[r] . x) for slot < n_slot, e = ids ? ids[slot] : slot
// With x1, slots from x_split on read x1 instead of x (two activation vectors in one launch).
hipError_t launch_moe_gateup(const ExpertSet &ex, const uint32_t *ids, uint32_t n_slot, uint32_t hidden, uint32_t ffn,
                             const float *x, float *act, hipStream_t s, const float *x1 = nullptr, uint32_t x_split = 0u);
// out[i] = sum_k weights[k] * tmp[k][row_start + i], k in order (tmp [top_k][hidden], i < row_count)
hipError_t launch_weighted_sum(const float *tmp, const float *weights, uint32_t top_k, uint32_t hidden, uint32_t row_start,
                               uint32_t row_count, float *out, hipStream_t s);

// out[r] = sum_k weights[k] * (down_{ids[k]}[r] . act[k]) + scalar[0] * (shared_down[r] . shared_act), k in selection order
hipError_t launch_moe_down_combine(const ExpertSet &ex, const uint32_t *ids, const float *weights, uint32_t top_k,
                                   const ExpertSet &shared, const float *scalar, uint32_t hidden, uint32_t ffn,
                                   const float *act, const float *shared_act, float *out, hipStream_t s);

// batched experts over pairs sorted by expert (the grouping below). uid / expert_start / n_unique on the device; n_groups
// is the launch bound on the number of groups (groups >= *n_unique exit at once). With uid == nullptr and
// expert_start == nullptr there is a single group (expert 0 of `ex`) whose pairs are tokens 0..n_pairs_total-1.
hipError_t launch_batch_gateup(const ExpertSet &ex, const uint32_t *uid, const uint32_t *expert_start, const uint32_t *pair_token,
                               const uint32_t *n_unique, uint32_t n_groups, uint32_t n_pairs_total, uint32_t hidden, uint32_t ffn,
                               const float *x, float *act, hipStream_t s);                     // act [pairs][ffn]
hipError_t launch_batch_down(const ExpertSet &ex, const uint32_t *uid, const uint32_t *expert_start, const uint32_t *n_unique,
                             uint32_t n_groups, uint32_t n_pairs_total, uint32_t hidden, uint32_t ffn, const float *act, float *tmp,
                             hipStream_t s);                                                    // tmp [pairs][hidden]
// out[t] = sum_k pair_weight[tok_pair[t][k]] * tmp[tok_pair[t][k]] (k in selection order) + scalar[t] * sh_tmp[t]
hipError_t launch_batch_combine(const float *tmp, const float *pair_weight, const uint32_t *tok_pair, uint32_t ntok, uint32_t top_k,
                                const float *sh_tmp, const float *scalar, uint32_t hidden, float *out, hipStream_t s);

// pair sort of [ntok][top_k] ids: see redhip_moe_group in include/redhip_moe.h
// f32 router logits of a chunk of tokens as a tiled fp32 MFMA product (every router row read once per 32 tokens), plus the
// fp16 split of the activations; same outputs as launch_router_gemv
// out[tok][row] = W[row] . x[tok] on the fp32 matrix units: W f32 [n_rows][K] (+ one optional extra row), x f32 [ntok][K]
hipError_t launch_f32_tiles(const float *w, const float *extra_row, const float *x, uint32_t ntok, uint32_t K, uint32_t n_rows, float *out,
                            uint32_t out_stride, void *xh, void *xl, int *xexp, hipStream_t s);
hipError_t launch_swiglu_rows(const float *gu, uint32_t gu_stride, uint32_t ntok, uint32_t ffn, float *act, hipStream_t s);
hipError_t launch_router_f32_tiles(const float *w, const float *gate_inp, const float *x, uint32_t ntok, uint32_t hidden, uint32_t n_expert,
                                   float *logits, void *xh, void *xl, int *xexp, hipStream_t s);
// prefill chunk on packed IQ2_XXS experts: tiles of 16 pairs per distinct expert, 16x16x16 fp16 MFMA. Needs the pair
// grouping (uid, expert_start, pair_token, n_unique); writes tmp [pairs][hidden] and sh_tmp [ntok][hidden] for
// launch_batch_combine. tile_* hold prefill_tile_bound() entries.
inline uint32_t prefill_tile_bound(uint32_t ntok, uint32_t top_k, uint32_t n_expert) {
    const uint32_t P = ntok * top_k;
    return (P < n_expert ? P : n_expert) + P / 16u + (ntok + 15u) / 16u + 1u;
}
// tiled_experts / tiled_shared: optional tile-major copies (launch_tile_packed) of the same matrices, same stride and offsets; with
// them and ffn <= 512 the kernels that keep a tile's activations in registers run.
hipError_t launch_tile_packed(const void *packed, uint64_t packed_stride, uint32_t count, uint32_t nrows, uint32_t K, void *tiled, uint64_t tiled_stride,
                              hipStream_t s, bool with_sc = false);
// routed gate/up + SwiGLU of a chunk on the tile-major copy of packed IQ2_XXS gate/up matrices (mixed layouts); act: f32 [pairs][ffn], or
// nullptr for fp16 halves + two exponents per pair in act_h / act_l / act_exp
hipError_t launch_prefill_gateup_tiled(const void *tiled_experts, uint64_t stride, const uint32_t *uid, const uint32_t *expert_start,
                                       const uint32_t *pair_token, const uint32_t *n_unique, uint32_t *tile_group, uint32_t *tile_pair0, uint32_t *tile_n,
                                       uint32_t *n_tiles, const void *xh, const void *xl, const int *xexp, float *act, void *act_h, void *act_l,
                                       int *act_exp, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert, hipStream_t s, bool tiles_built = false);      // tiles_built: launch_group_pairs wrote the tile lists
// tile-major IQ3_S matrices (one 32-bit word per eight weights) from raw GGUF rows, and the routed down projection of a chunk on them
hipError_t launch_tile_iq3s(const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K, void *tiled, uint64_t tiled_stride, hipStream_t s);
// routed matrices of a chunk whose experts are IQ2_XS / IQ1_M: tile kernels on the row-major streams (gate | up at `packed`, down at `down`)
hipError_t launch_prefill_streams(uint32_t gate_up_type, const int8_t *gate_up_grid, const void *packed, uint64_t packed_stride, uint32_t down_type,
                                  const int8_t *down_grid, const void *down, uint64_t down_stride, const uint32_t *uid, const uint32_t *expert_start,
                                  const uint32_t *pair_token, const uint32_t *n_unique, uint32_t *tile_group, uint32_t *tile_pair0, uint32_t *tile_n,
                                  uint32_t *n_tiles, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l, int *act_exp, float *tmp,
                                  uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert, hipStream_t s, bool tiles_built = false);      // tiles_built: launch_group_pairs wrote the tile lists
hipError_t launch_prefill_down_iq3s(const void *tiled_down, uint64_t stride, const uint32_t *uid, const uint32_t *n_unique, const uint32_t *tile_group,
                                    const uint32_t *tile_pair0, const uint32_t *tile_n, const uint32_t *n_tiles, const void *act_h, const void *act_l,
                                    const int *act_exp, float *tmp, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert,
                                    hipStream_t s);
hipError_t launch_prefill_packed(const void *experts, uint64_t stride, const void *shared, const void *tiled_experts, const void *tiled_shared,
                                 const uint32_t *uid, const uint32_t *expert_start,
                                 const uint32_t *pair_token, const uint32_t *n_unique, uint32_t *tile_group, uint32_t *tile_pair0,
                                 uint32_t *tile_n, uint32_t *n_tiles, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l,
                                 int *act_exp, float *tmp, float *sh_tmp, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok,
                                 uint32_t n_expert, hipStream_t s, bool tiles_built = false, bool with_shared = true);      // without: no shared expert's tiles (shared, tiled_shared, sh_tmp unused)      // tiles_built: launch_group_pairs wrote the tile lists
// Tile lists of a chunk for the prefill kernels. Groups 0..U-1 are the distinct routed experts (pairs expert_start[u] ..
// expert_start[u + 1]), group U is the shared expert with pairs P .. P + shared_ntok (0: no shared tiles). A tile = (group, first pair,
// number of pairs). Three lists in the same arrays, list l from entry l * list_stride on (list_stride = prefill_tile_bound of the call),
// its length in n_tiles[l]:
//   0  tiles of kPrefillTile pairs (the down kernels; the gate/up kernel of hidden 512)
//   1  "wide" tiles of 17 .. kPrefillWideTile pairs: a group's runs of 32 pairs, and its remainder when that is more than 16
//   2  "narrow" tiles: the remainders of 1 .. 16 pairs
// Lists 1 and 2 together cover every pair once: the gate/up kernel takes the wide tiles on the path that multiplies two sets of 16 pairs
// with every decoded weight, the narrow ones on the path for 16.
constexpr uint32_t kPrefillTile = 16u, kPrefillWideTile = 32u;
struct TileLists {
    uint32_t *tile_group, *tile_pair0, *tile_n, *n_tiles;
    uint32_t list_stride, shared_ntok;
};
#ifdef __HIPCC__
// By all 1024 threads of one workgroup: thread u < U brings its group's run (first pair p0, n pairs), the others n = 0; wave_total:
// LDS scratch. Exclusive prefix sums of the tiles per group, then every group writes its tiles.
__device__ __forceinline__ void build_tile_lists(uint32_t U, uint32_t p0, uint32_t n, uint32_t P, const TileLists &tl, uint32_t (*wave_total)[16]) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    auto counts = [](uint32_t m, uint32_t *c) {            // tiles of m pairs in the three lists
        const uint32_t rem = m % kPrefillWideTile;
        c[0] = (m + kPrefillTile - 1u) / kPrefillTile;
        c[1] = m / kPrefillWideTile + (rem > kPrefillTile ? 1u : 0u);
        c[2] = rem > 0u && rem <= kPrefillTile ? 1u : 0u;
    };
    uint32_t mine[3], scan[3];
    counts(n, mine);
#pragma unroll
    for (int l = 0; l < 3; ++l) {
        scan[l] = mine[l];
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = __shfl_up(scan[l], o, 64);
            if (lane >= (uint32_t)o) scan[l] += up;
        }
        if (lane == 63u) wave_total[l][wave] = scan[l];
    }
    __syncthreads();
    uint32_t sh[3];
    counts(tl.shared_ntok, sh);
#pragma unroll
    for (int l = 0; l < 3; ++l) {
        uint32_t base = 0u, routed_tiles = 0u;
        for (uint32_t w = 0; w < 16u; ++w) { if (w < wave) base += wave_total[l][w]; routed_tiles += wave_total[l][w]; }
        const uint32_t off = (uint32_t)l * tl.list_stride, first = off + base + scan[l] - mine[l];
        // tile t of a run of m pairs that starts at pair q0, in list l
        auto put = [&](uint32_t at, uint32_t group, uint32_t q0, uint32_t m, uint32_t t) {
            const uint32_t size = l == 0 ? kPrefillTile : kPrefillWideTile, start = l == 2 ? m - m % kPrefillWideTile : size * t;
            tl.tile_group[at] = group;
            tl.tile_pair0[at] = q0 + start;
            tl.tile_n[at] = m - start < size ? m - start : size;
        };
        for (uint32_t t = 0; t < mine[l]; ++t) put(first + t, tid, p0, n, t);
        for (uint32_t t = tid; t < sh[l]; t += 1024u) put(off + routed_tiles + t, U, P, tl.shared_ntok, t);
        if (tid == 0u) tl.n_tiles[l] = routed_tiles + sh[l];
    }
}
#endif
// Device scratch of the pair sort of large chunks (more than 512 tokens), which runs as three launches over blocks of kGroupSpan tokens:
// count_blk / blk_off [blocks][n_expert], first_key / expert_base [n_expert]. All zero before the first use (the sort leaves first_key
// zero again); `blocks` = the capacity in blocks.
constexpr uint32_t kGroupSpan = 64u;
struct GroupScratch { uint32_t *count_blk, *blk_off, *first_key, *expert_base; uint32_t blocks; };
inline size_t group_scratch_bytes(uint32_t max_tokens, uint32_t n_expert) {
    return sizeof(uint32_t) * ((size_t)2u * ((max_tokens + kGroupSpan - 1u) / kGroupSpan) + 2u) * n_expert;
}
inline GroupScratch group_scratch_at(void *base, uint32_t max_tokens, uint32_t n_expert) {
    const uint32_t nb = (max_tokens + kGroupSpan - 1u) / kGroupSpan;
    uint32_t *p = static_cast<uint32_t *>(base);
    return GroupScratch{p, p + (size_t)nb * n_expert, p + (size_t)2u * nb * n_expert, p + (size_t)2u * nb * n_expert + n_expert, nb};
}
// tiles: also write the tile lists of the chunk (the prefill launchers then take tiles_built = true and launch no build_tiles_kernel)
// scratch: when given, chunks of more than 512 tokens are sorted by many workgroups (three launches) instead of one
hipError_t launch_group_pairs(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t n_expert,
                              uint32_t *uid, uint32_t *expert_start, uint32_t *pair_token, float *pair_weight,
                              uint32_t *tok_pair, uint32_t *n_unique, hipStream_t s, const TileLists *tiles = nullptr, const GroupScratch *scratch = nullptr);

// ---- decode path over packed IQ2_XXS (redhip_fused.hip) ----

// shapes the packed kernels tile: gate/up rows in chunks of 512 columns over 16 waves; down rows of <= 1024 columns
inline bool fused_iq2_supported(uint32_t hidden, uint32_t ffn) {
    const uint32_t nkc = hidden / 512u;
    return hidden % 512u == 0u && (nkc == 1u || nkc == 2u || nkc == 4u || nkc == 8u) && ffn && ffn % 256u == 0u && ffn <= 1024u;
}

// `count` matrices, raw_stride / packed_stride bytes apart; packed = qs [nrows][K/32] uint2 then ds [nrows][K/256] fp16
hipError_t launch_repack_iq2xxs(const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K, bool col_major,
                                void *packed, uint64_t packed_stride, hipStream_t s);
// gate / up matrices of IQ2_XXS, IQ2_XS or IQ1_M rows into the streams of the one-token gate/up kernel (col_major: every array
// [group or block][row] instead of [row][group or block], the column-sliced form of a down matrix)
hipError_t launch_repack_gateup(uint32_t type, const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K,
                                void *packed, uint64_t packed_stride, hipStream_t s, bool col_major = false);
// bytes of one such matrix: 8 per 32 weights + 2 per 256, IQ2_XS one more per 32
inline uint64_t packed_matrix_bytes(uint32_t type, uint32_t nrows, uint32_t K) {
    return (uint64_t)nrows * ((uint64_t)(K / 32u) * (type == T_IQ2_XS ? 9u : 8u) + (uint64_t)(K / 256u) * 2u);
}
hipError_t launch_dequant_packed(uint32_t type, const void *packed, uint32_t nrows, uint32_t K, const int8_t *grid, float *out, hipStream_t s, bool col_major = false);
hipError_t launch_dequant_packed_iq2xxs(const void *packed, uint32_t nrows, uint32_t K, bool col_major, float *out, hipStream_t s);

// Pair sort of caller-given routing (at most 16 tokens, 256 pairs, 1024 experts) as a side job of another launch: one extra
// workgroup groups ids / weights [ntok][top_k] by expert while the others do the launch's own work. Outputs as launch_group_pairs.
struct GroupJob {
    const uint32_t *ids;
    const float *weights;
    uint32_t ntok, top_k, n_expert;
    uint32_t *uid, *expert_start, *pair_token;
    float *pair_weight;
    uint32_t *tok_pair, *n_unique;
    uint32_t *status = nullptr;      // RouteGuard::status of the call (ids are clamped to n_expert - 1 either way)
    uint2 *pass_list = nullptr;      // optional: the pass list of the batched expert-slice kernel, at most ntok * top_k entries, and
    uint32_t *n_pass = nullptr;      // their number
};

// the pair sort (and pass list) of a caller's routing as one launch: up to 32 tokens and 512 pairs
hipError_t launch_group_small(const GroupJob &job, hipStream_t s);

// Selection inside the batched gate/up kernel: logits [ntok][n_expert + 1] in, the routing out (ids, weights [ntok][top_k], scalar [ntok]);
// the grouping arrays handed to the launcher are then outputs too.
struct BatchSelect {
    const float *logits;
    uint32_t n_expert;
    uint32_t *ids;
    float *weights;
    float *scalar;
};

// logits [ntok][n_expert + 1] (entry n_expert = gate_inp . x) and the fp16 split of x: xh, xl [ntok][hidden], xexp [ntok]
// sh_dense: f32 [2 ffn][hidden] shared gate | up rows (F32 router, <= 8 tokens). job / job_done: the launch carries the pair sort
// when its kernel can (*job_done says whether it did).
hipError_t launch_router_gemv(uint32_t router_type, const void *w, const float *x, const float *gate_inp, uint32_t ntok, uint32_t hidden,
                              uint32_t n_expert, float *logits, void *xh, void *xl, int *xexp, const void *sh_q6k, float *sh_gu, uint32_t ffn,
                              hipStream_t s, const float *sh_dense = nullptr, float *scalar_out = nullptr, const GroupJob *job = nullptr,
                              bool *job_done = nullptr);
// softmax top-k of logits [ntok][n_expert + 1]; scalar[t] = sigmoid(logits[t][n_expert]); optional probs [ntok][n_expert]
hipError_t launch_select(const float *logits, uint32_t ntok, uint32_t n_expert, uint32_t top_k, uint32_t *ids, float *weights, float *scalar,
                         float *probs, hipStream_t s);
// 2..8 tokens: softmax top-k per token and the pair sort (outputs of `job`, pass list included) in one launch of one workgroup
hipError_t launch_select_group(const float *logits, uint32_t ntok, uint32_t n_expert, uint32_t top_k, uint32_t *ids, float *weights, float *scalar,
                               const GroupJob &job, hipStream_t s);
// fp16 split of x and the scalar gate without a router; with a job that fits, one more workgroup does the pair sort (*job_done)
hipError_t launch_prep(const float *x, const float *gate_inp, uint32_t ntok, uint32_t hidden, void *xh, void *xl, int *xexp, float *scalar, hipStream_t s,
                       const GroupJob *job = nullptr, bool *job_done = nullptr);

// single token: act[slot] = SwiGLU(gate . x, up . x) as fp16 halves with one exponent per 32 values. With `logits` the
// kernel selects the experts itself (and writes ids / weights / scalar); with logits == nullptr it takes ids_in.
hipError_t launch_gateup_select(const void *experts, uint64_t stride, const void *shared, const void *shared_q6k, const float *x,
                                const float *shared_gu, const float *logits, const uint32_t *ids_in, uint32_t *ids_out, float *weights_out,
                                float *scalar_out, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l, int *act_exp,
                                uint32_t hidden, uint32_t ffn, uint32_t n_expert, uint32_t top_k, hipStream_t s, uint32_t ntok = 1u,
                                uint32_t gate_up_type = T_IQ2_XXS, const int8_t *grid = nullptr);
// small batch on a mixed layout with the pairs grouped by expert: batched MFMA gate/up on the packed IQ2_XXS / IQ2_XS / IQ1_M matrices
// (shared expert's products given), batched MFMA down on the packed copy (`words_down`: IQ3_S words or the streams of the other three
// formats) with the shared rows from `dense_down`, else batched raw-row down of the built-in block types; every distinct expert is read once
hipError_t launch_batch_mixed(uint32_t gate_up_type, const int8_t *gate_up_grid, const void *packed, uint64_t packed_stride, const float *shared_gu,
                              uint32_t down_type, const int8_t *down_grid, uint32_t shared_down_type,
                              const void *raw_down, uint64_t raw_stride, const void *shared_down, const void *words_down, uint64_t words_stride,
                              const float *dense_down, const uint32_t *uid, const uint32_t *expert_start,
                              const uint32_t *pair_token, const uint32_t *n_unique, const float *pair_weight, const uint32_t *tok_pair,
                              const float *scalar, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l, int *act_exp,
                              float *out, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert, hipStream_t s,
                              const BatchSelect *select = nullptr);
// IQ3_S down matrices of mixed layouts as one word per eight weights (uint4 per 32, [row][K/32], then d as fp16 [row][K/256])
hipError_t launch_repack_iq3s_words(const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K, void *packed, uint64_t packed_stride, hipStream_t s,
                                    bool col_major = false);      // col_major: words [K / 32][nrows], d [K / 256][nrows]
hipError_t launch_dequant_iq3s_words(const void *packed, uint32_t nrows, uint32_t K, float *out, hipStream_t s, bool col_major = false);
inline uint64_t iq3s_words_bytes(uint32_t nrows, uint32_t K) { return (uint64_t)nrows * ((uint64_t)(K / 32u) * 16u + (uint64_t)(K / 256u) * 2u); }
// down + combine of one token (ntok > 1: one grid layer per token) on word-packed IQ3_S routed matrices and the shared expert's dense f32 copy
// (IQ2_XS / IQ1_M down matrices: the streams of launch_repack_gateup and the caller's codebook)
hipError_t launch_down_combine_words(uint32_t down_type, const int8_t *grid, const void *experts, uint64_t stride, const float *shared_dense, const uint32_t *ids,
                                     const float *weights, const float *scalar, const void *act_h, const void *act_l, const int *act_exp, float *out,
                                     uint32_t hidden, uint32_t ffn, uint32_t top_k, hipStream_t s, uint32_t ntok = 1u,
                                     bool col_major = false);      // col_major (IQ3_S): the column-sliced copy of launch_repack_iq3s_words
// down + weighted combine for layouts whose down matrices are raw GGUF rows of any supported type
hipError_t launch_down_combine_raw(uint32_t down_type, uint32_t shared_down_type, const void *experts, uint64_t stride, const void *shared,
                                   const uint32_t *ids, const float *weights, const float *scalar, const void *act_h, const void *act_l,
                                   const int *act_exp, float *out, uint32_t hidden, uint32_t ffn, uint32_t top_k, hipStream_t s, uint32_t ntok = 1u,
                                   const int8_t *grid = nullptr, const float *shared_dense = nullptr);
// single token on all-IQ2_XXS layers, two launches: expert slices (selection from `logits`, or the caller's ids_in / weights_in / scalar_in;
// gate / up / SwiGLU / the matching columns of the down matrix from its column-sliced copy; partial [top_k + 1][ffn / 32][hidden]), then
// the sum of the partial vectors into out [hidden]
hipError_t launch_expert_slices(const void *experts, uint64_t stride, const void *down_cm, uint64_t down_stride, const void *shared, const void *shared_down_cm,
                                const float *logits, const uint32_t *ids_in, const float *weights_in, const float *scalar_in, uint32_t *ids_out,
                                float *weights_out, float *scalar_out, const void *xh, const void *xl, const int *xexp, float *partial, float *out,
                                uint32_t hidden, uint32_t ffn, uint32_t n_expert, uint32_t top_k, hipStream_t s, const float *shared_gu = nullptr,
                                const float *shared_dense = nullptr, uint32_t stream_type = 0u, const int8_t *grid = nullptr);
// (shared_gu and shared_dense given: a mixed layout as launch_batch_slices takes it - down_cm holds column-sliced word-packed IQ3_S, or with
// stream_type IQ2_XS / IQ1_M and the codebook `grid`, experts / down_cm hold the row-major / column-sliced streams; the shared expert is dense)
// one token over slots of a pool whose re-laid IQ2_XXS copies (packed gate | up, column-sliced down) lie shadow_off behind the raw bytes
// that slot_table [top_k] points at; x split to fp16 halves inside the kernel (experts from x_split on read x1 when given); partial
// [top_k][ffn / 32][hidden]; with tail_resid: out = tail_out2 = tail_resid + (sum + tail_shared * tail_scalar[0]). top_k <= 64
hipError_t launch_slot_slices(const uint64_t *slot_table, uint64_t shadow_off, const float *weights, uint32_t top_k, uint32_t hidden, uint32_t ffn,
                              const float *x, const float *x1, uint32_t x_split, float *partial, float *out, const float *tail_resid,
                              const float *tail_shared, const float *tail_scalar, float *tail_out2, hipStream_t s, uint32_t kind = 0u,
                              const int8_t *grid = nullptr);
// (kind 1: the copies hold packed IQ2_XXS gate | up and column-sliced IQ3_S words; 2 / 3: row-major IQ2_XS / IQ1_M streams of gate | up,
// column-sliced streams of down, decoded through the codebook `grid`; kinds 1..3: hidden <= 2048)
// the same for 2..32 tokens (at most 512 pairs) whose pairs are grouped by expert: pass_list / n_pass from the pair sort (GroupJob), weights
// [ntok][top_k] and scalar [ntok] of the routing; partial [ntok][top_k + 1][ffn / 32][hidden]
hipError_t launch_batch_slices(const void *experts, uint64_t stride, const void *down_cm, uint64_t down_stride, const void *shared, const void *shared_down_cm,
                               const void *pass_list, const uint32_t *n_pass, const float *weights, const float *scalar, const void *xh, const void *xl,
                               const int *xexp, float *partial, float *out, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, hipStream_t s,
                               const float *shared_gu = nullptr, const float *shared_dense = nullptr, uint32_t stream_type = 0u, const int8_t *grid = nullptr);
// (with shared_gu / shared_dense: a mixed layout - gate / up packed IQ2_XXS in `experts`, down_cm column-sliced word-packed IQ3_S, the shared
// expert as its gate | up products [ntok][2 ffn] and the dense f32 copy [hidden][ffn] of its down matrix; shared / shared_down_cm unused.
// With stream_type IQ2_XS / IQ1_M and the caller's codebook besides: `experts` and down_cm hold that format's streams, down_cm column-sliced)

}  // namespace redhip
