/*
 * Resident MoE FFN layers - C ABI of libredmetal_hip.so (MI355X / gfx950).
 *
 * The production path: every expert of every layer stays in HBM, and one call runs the whole FFN of a layer
 * for 1..max_tokens tokens on a HIP stream without touching the host:
 *   router GEMV -> softmax top-k -> (token grouping) -> routed experts -> shared expert -> combine.
 * It stands where the reference has the resident top-k pool with its residency table and stream-encoded
 * execution (native/redmetal_topk.h:107-170, encode_device / encode_device_tail / encode_batched) driven by
 * emit_ffn_pre_opt + emit_layer_experts (native/redmetal_engine.m:1733-1765,1800-1863) and, for chunks,
 * prefill_chunk (native/redmetal_engine_prefill.m:1238-1300). The opaque Metal objects of those calls
 * (id<MTLCommandBuffer>, id<MTLBuffer>) become a hipStream_t and device pointers.
 *
 * Conventions follow the pool families: int 1 = success / 0 = failure, message via redhip_moe_last_error()
 * (thread-local), abi_version() == 1, handles made and destroyed by the caller, destroy(NULL) is a no-op.
 * `*_dev` arguments are device pointers; `stream` is a hipStream_t (NULL = the default stream). Calls that
 * take a stream only enqueue work. One forward at a time per handle: the handle owns the workspace.
 * Chunks (more than 8 tokens) on mixed-precision layouts run part of their work on a second stream that the
 * handle owns, forked from `stream` and joined to it again with events inside the same call (capturable).
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *redhip_moe_t;

typedef struct {
    uint32_t hidden;            /* multiple of 256 */
    uint32_t ffn;               /* multiple of 256 */
    uint32_t n_expert;          /* <= 1024 */
    uint32_t top_k;             /* <= 16 (the one-token and small-batch MFMA kernels serve 2..15, other values run on the generic kernels) */
    uint32_t n_layer;
    uint32_t max_tokens;        /* largest ntok of redhip_moe_forward (the reference's prefill hands over chunks of up to 2048 tokens,
                                   native/redmetal_engine_prefill.m:1246-1277). It also decides which copies of the weights the handle keeps
                                   beside the raw blocks: 1 - the streams of the one-token kernels; 2..8 - also the column-sliced down copy of
                                   the small-batch kernels; more than 8 - also the tile-major copies of the chunk kernels */
    uint32_t router_type;       /* 0 (F32) or 14 (Q6_K) */
    uint32_t expert_type_word;  /* gate_up | down << 8, as native/redlite_native_metal.h:69-73; types 16 (IQ2_XXS), 21 (IQ3_S), 14 (Q6_K), and
                                   17 (IQ2_XS) / 29 (IQ1_M) after redhip_set_codebooks */
    uint32_t shared_type_word;  /* same encoding for the shared expert; types 16, 21, 14 */
    uint32_t reserved;
} redhip_moe_config;

uint32_t redhip_moe_abi_version(void);
const char *redhip_moe_last_error(void);

redhip_moe_t redhip_moe_create(const redhip_moe_config *config);
void redhip_moe_destroy(redhip_moe_t moe);
uint64_t redhip_moe_resident_bytes(redhip_moe_t moe);     /* weight bytes held in HBM */

/* One-time uploads of raw GGUF blocks (the layout of native/redlite_native_gguf.c:402-440: rows back to back,
 * experts contiguous). Sources may be host or device memory. Synchronous. */
int redhip_moe_load_router(redhip_moe_t moe, uint32_t layer, const void *weights, uint64_t bytes);
int redhip_moe_load_shared(redhip_moe_t moe, uint32_t layer, const float *gate_inp,
    const void *gate, uint64_t gate_bytes, const void *up, uint64_t up_bytes, const void *down, uint64_t down_bytes);
int redhip_moe_load_experts(redhip_moe_t moe, uint32_t layer, uint32_t first_expert, uint32_t count,
    const void *gate, const void *up, const void *down);   /* count experts, each tightly packed */

/* out_dev[t][hidden] = routed(x_t) + shared(x_t) * sigmoid(gate_inp . x_t), t < ntok. x_dev is [ntok][hidden]
 * f32. Stream-ordered, no host synchronisation. */
int redhip_moe_forward(redhip_moe_t moe, uint32_t layer, const float *x_dev, uint32_t ntok, float *out_dev, void *stream);

/* Stream-ordered pieces of the same path (what forward chains), for callers that interleave their own work and
 * for parity taps. ids_dev [ntok][top_k] u32, weights_dev [ntok][top_k] f32, logits_dev [ntok][n_expert] f32.
 * Contract of routing a caller hands in (redhip_moe_experts, redhip_moe_group), as the reference checks its host-side lists
 * (native/redmetal_topk.m:1313,1635-1636): every id < n_expert, and the ids of one token distinct. The ids live in device memory
 * and cannot be checked before the kernels run, so the kernels guard themselves: an id >= n_expert is clamped to n_expert - 1
 * (no out-of-bounds access), and both violations set a status word that makes the next redhip_moe_last_route on the handle fail
 * with a message (and clears it). Outputs of a call that broke the contract are not meaningful. */
int redhip_moe_route(redhip_moe_t moe, uint32_t layer, const float *x_dev, uint32_t ntok,
    uint32_t *ids_dev, float *weights_dev, float *logits_dev, void *stream);
int redhip_moe_experts(redhip_moe_t moe, uint32_t layer, const float *x_dev, uint32_t ntok,
    const uint32_t *ids_dev, const float *weights_dev, float *out_dev, void *stream);

/* Routing of the last forward / route on this handle, copied to host after synchronising `stream`. Any may be NULL. Fails (0, message)
 * when a call since the last one was given routing that broke the contract above. */
int redhip_moe_last_route(redhip_moe_t moe, uint32_t ntok, uint32_t *ids, float *weights, float *logits, void *stream);

/* GGUF side (the role of native/redlite_native_gguf.c:196-440 and the tensor checks of
 * native/redlite_native_engine.c:170-179): the MoE tensors of layer `first_layer + l` are blk.N.ffn_gate_inp.weight
 * (router, (hidden, experts)), ffn_gate_inp_shexp.weight (F32 [hidden]), ffn_{gate,up,down}_shexp.weight and the
 * expert-major ffn_{gate,up,down}_exps.weight ((hidden, ffn, experts) resp. (ffn, hidden, experts)).
 * redhip_gguf_moe_config fills hidden / ffn / n_expert / top_k (from <arch>.expert_used_count) / types / n_layer (the
 * run of consecutive MoE layers from first_layer that share its shapes and quantisation types: a file that changes its
 * expert format between layers is walked as one run, and one handle, per format) and max_tokens = 1 from a GGUF v2 /
 * v3 file;
 * redhip_moe_load_gguf uploads layers first_layer .. first_layer + n_layer - 1 of the file into layers 0 .. of a
 * handle created with `cfg`. Errors: return 0 and redhip_gguf_last_error() (thread-local). */
const char *redhip_gguf_last_error(void);
int redhip_gguf_moe_config(const char *path, uint32_t first_layer, redhip_moe_config *out);
int redhip_moe_load_gguf(redhip_moe_t moe, const char *path, uint32_t first_layer, uint32_t n_layer, const redhip_moe_config *cfg);

/* Where the bytes of one routed expert lie in the file: the answer of rl_native_build_expert_map + rl_native_expert_layout
 * (native/redlite_native_gguf.c:199-397 and :399-440; struct rl_expert_layout of native/redlite_native_gguf.h:47-59, same
 * fields in the same order) as this library's reader sees the file, i.e. the byte ranges redhip_moe_load_gguf uploads.
 * Offsets are absolute file offsets. `expected_experts` is checked against the last dimension of the three tensors.
 * Fails (0, redhip_gguf_last_error) for an expert beyond the count, a layer without its gate / up / down tensors, or gate
 * and up tensors of different types, as the reference does. Host code only: no GPU is touched. */
typedef struct {
    uint32_t layer;
    uint32_t expert;
    uint32_t ggml_type;      /* gate and up */
    uint32_t down_type;
    uint64_t gate_offset, gate_bytes;
    uint64_t up_offset, up_bytes;
    uint64_t down_offset, down_bytes;
    uint64_t total_bytes;
} redhip_gguf_expert_layout_t;
int redhip_gguf_expert_layout(const char *path, uint32_t expected_experts, uint32_t layer, uint32_t expert, redhip_gguf_expert_layout_t *out);

/* The layer with the steps on either side of it, one call per layer and token batch
 * (native/redlite_native_engine_cpu.c:418-427; Metal rl_resid_rms native/redmetal_engine.m:95-105 in front and
 * rl_moe_tail :61-69 behind): resid = x + branch (the attention / DeltaNet branch output), the layer's input is
 * resid * rsqrt(mean(resid^2) + eps) * post_norm, and x_out = resid + layer output. All pointers are device
 * memory, [ntok][hidden] except post_norm_dev [hidden]; x_out_dev may be x_dev. Enqueues kernels only. Where the
 * path allows, the norm is computed inside the router launch and the residual is added by the last kernel, so the
 * two extra launches of the reference disappear. */
int redhip_moe_forward_block(redhip_moe_t moe, uint32_t layer, const float *x_dev, const float *branch_dev,
    const float *post_norm_dev, float eps, uint32_t ntok, float *x_out_dev, void *stream);

/* Token grouping of [ntok][top_k] ids (device), the GPU form of the pair sort in
 * native/redmetal_engine_prefill.m:1246-1276: uid_dev[U] in first-appearance order, expert_start_dev[U+1],
 * pair_token_dev[P], pair_weight_dev[P], tok_pair_dev[P], n_unique_dev[1]; P = ntok * top_k. */
int redhip_moe_group(redhip_moe_t moe, const uint32_t *ids_dev, const float *weights_dev, uint32_t ntok,
    uint32_t *uid_dev, uint32_t *expert_start_dev, uint32_t *pair_token_dev, float *pair_weight_dev,
    uint32_t *tok_pair_dev, uint32_t *n_unique_dev, void *stream);

/* The int8 codebooks of IQ2_XS (512 x 8) and IQ1_M (2048 x 8) that type 17 / 29 rows decode through, copied to the device
 * for the taps below; either may be NULL to keep what is there. The reference hands the same two tables to
 * redmetal_ffn_pool_create and redmetal_quant_rows (native/redmetal_ffn.h:9-18, native/redmetal_quant.h:9-27), which upload
 * them too. Process-wide and synchronous: the process holds one pair of tables. Resident layers with such experts, and pools that have run
 * one, are bound to the tables' content: while any of them is alive, a call (here, or through a pool / redmetal_quant_rows) that brings
 * different tables fails with a message instead of changing what they decode through; the same content again is free. */
int redhip_set_codebooks(const int8_t *iq2_xs_grid, uint32_t iq2_xs_count, const int8_t *iq1_m_grid, uint32_t iq1_m_count);

/* Parity tap: f32 dequantisation of `rows` rows of `ncols` weights of raw GGUF blocks (device pointers). */
int redhip_dequant_rows(uint32_t ggml_type, const void *rows_dev, uint32_t nrows, uint32_t ncols, float *out_dev, void *stream);
/* Parity tap: dequantise one resident matrix (which: 0 gate, 1 up, 2 down; expert == n_expert: shared expert;
 * which == 3: the router; which == 4: the down matrix from the column-sliced copy that the expert-slice kernels read - all-IQ2_XXS
 * layers, and the routed experts of layers with IQ2_XXS gate/up and IQ3_S down matrices or with every routed matrix IQ2_XS or IQ1_M)
 * from the layout the kernels read.
 * out_dev holds rows x cols floats. */
int redhip_moe_dequant_resident(redhip_moe_t moe, uint32_t layer, uint32_t expert, uint32_t which, float *out_dev, void *stream);

/* GEMV on device memory: out_dev[r] = W[row_start + r] . x_dev, raw GGUF rows. */
int redhip_gemv_rows(uint32_t ggml_type, const void *matrix_dev, uint32_t ncols, uint32_t row_start, uint32_t row_count,
    const float *x_dev, float *out_dev, void *stream);

/* Per-stage kernel timing, the counterpart of the reference's RL_ENGINE_PROFILE stage timers
 * (native/redmetal_engine.m:1150-1164). Between begin and end every kernel this library launches is bracketed
 * by events that take the dispatch's own begin/end timestamps; end synchronises the device and returns, per
 * stage, the summed kernel time in ms and the number of launches. Process-wide, for benchmarks. */
uint32_t redhip_profile_stage_count(void);
const char *redhip_profile_stage_name(uint32_t stage);
int redhip_profile_begin(void);
int redhip_profile_end(double *stage_ms, uint32_t *stage_launches, uint32_t n_stage);
/* Phase stamps inside the expert kernels (no counterpart in the reference's C surface; its RL_ENGINE_PROFILE stops at whole stages): a
 * library built with -DREDHIP_TIMELINE (python dwarfstar_red_lite_amd/build.py --timeline) stores, per workgroup of the last expert launch,
 * the 100 MHz wall clock at every phase boundary: stamps[workgroup * 16 + slot], slot 15 = the compute unit. Synchronises the device.
 * Returns 0 in an ordinary build. */
int redhip_timeline_read(uint64_t *stamps, uint32_t n_groups, uint32_t clear);
/* Counter calibration (no counterpart in the reference): one plain copy kernel, dst_dev[i] = src_dev[i] for
 * `bytes` bytes (a multiple of 16), reading and writing exactly that much. Memory-traffic counters collected for
 * the kernels above are scaled by what they read for this kernel of known size. */
int redhip_calibration_copy(void *dst_dev, const void *src_dev, uint64_t bytes, void *stream);
/* The machine's own yardsticks (the counterpart of the reference's kernel-bench, native/redmetal_engine_selftest.m:295-462): a
 * streaming read of `bytes` bytes (a multiple of 16; nothing is written; sink_dev: four bytes of device memory), and a dense fp16
 * matrix-core loop on register operands (`grid` workgroups of four waves, `iters` rounds of eight 16x16x32 MFMAs per wave;
 * *flops = what the launch computes). Time them with events around the call or with the stage profile above. */
int redhip_calibration_read(const void *src_dev, uint64_t bytes, void *sink_dev, void *stream);
int redhip_calibration_mfma(uint32_t grid, uint32_t iters, void *sink_dev, uint64_t *flops, void *stream);
/* Launch-cost calibration (no counterpart in the reference): one launch of `grid` workgroups of `block` lanes of a kernel that does
 * nothing. A chain of such launches with a path's grids is the time the path's dependent launches cost before any work. */
int redhip_calibration_empty(uint32_t grid, uint32_t block, void *stream);

#ifdef __cplusplus
}
#endif
