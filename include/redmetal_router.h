/*
 * Router - C ABI of libredmetal_hip.so (MI355X / gfx950).
 *
 * Replaces the router surface of native/redlite_native_router_exec.h:12-49. Error convention of this family:
 * caller-supplied `char *error, size_t error_cap`, set to "" on success; return 1 / 0.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RL_ROUTER_MAX_DIMS 8u

/* native/redlite_native_router.h:13-20 (same field order and widths) */
typedef struct {
    uint32_t layer;
    uint32_t ggml_type;
    uint32_t n_dims;
    uint64_t shape[RL_ROUTER_MAX_DIMS];     /* (hidden, experts) */
    uint64_t tensor_offset;
    uint64_t tensor_span_bytes;
} rl_router_tensor_info;

/* native/redlite_native_router_exec.h:12-15 */
typedef struct {
    double read_ms;
    double compute_ms;
} rl_native_router_telemetry;

/* native/redlite_native_router_exec.h:38-49, native/redmetal_router.m:22-171: logits[e] = W[e] . x from the
 * tensor at tensor_offset of the file. The reference accepts F32 only; Q6_K (14) is accepted as well. */
int rl_native_router_gpu_f32(const char *model_path, const rl_router_tensor_info *router,
    const float *input, uint32_t input_count, float *logits, uint32_t logits_count,
    rl_native_router_telemetry *telemetry, char *error, size_t error_cap);

/* native/redlite_native_router_exec.h:28-36, native/redlite_native_router_exec.c:102-184: softmax over all
 * experts, top_k by probability (ties to the lower index), weights renormalised over the selection. Runs on the
 * GPU (the kernel the resident layer path uses); probabilities may be NULL. */
int rl_native_router_select_softmax_topk(const float *logits, uint32_t expert_count, uint32_t top_k,
    uint32_t *expert_ids, float *router_weights, float *probabilities, char *error, size_t error_cap);

#ifdef __cplusplus
}
#endif
