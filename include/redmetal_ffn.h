/*
 * Single-expert FFN pool - C ABI of libredmetal_hip.so (MI355X / gfx950).
 *
 * Replaces the pool the reference declares in native/redmetal_ffn.h:9-70 and implements in
 * native/redmetal_ffn.m:425-706. Names, argument meaning, return convention (1 = success, 0 = failure,
 * message through redmetal_ffn_last_error(), thread-local) and the slot layout gate|up|down are kept, so a
 * caller of the reference binds this library unchanged. Differences, all additive:
 *   - ggml_type accepts the reference's IQ2_XS (17) / IQ1_M (29), decoded through the two codebooks handed to pool_create
 *     exactly as the reference takes them (non-NULL, exact counts, native/redmetal_ffn.m:223-227), plus IQ2_XXS (16),
 *     IQ3_S (21), Q6_K (14), whose tables are built in, and the reference's two-type word gate_up | down << 8
 *     (native/redlite_native_metal.h:69-73) mixing any of them.
 *   - the process holds one device copy of the two codebooks: a pool binds to their content the first time it runs an
 *     IQ2_XS / IQ1_M expert, and while bound pools or resident layers are alive a pool with different tables fails with a
 *     message instead of decoding through the wrong ones (the reference keeps two buffers per pool).
 *   - slots live in device memory (HBM); load_expert reads the file into pinned host memory and copies.
 * All pointers are host pointers; every call is synchronous.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *redmetal_ffn_pool_t;

/* native/redmetal_ffn.h:11-12, native/redmetal_ffn.m:424-427 */
uint32_t redmetal_ffn_abi_version(void);
const char *redmetal_ffn_last_error(void);

/* native/redmetal_ffn.h:14-22, native/redmetal_ffn.m:211-316,429-450. slot size is rounded up to 4096;
 * capacity = budget / slot size; slabs of slots_per_slab (0 = 64) slots are allocated on first use. */
redmetal_ffn_pool_t redmetal_ffn_pool_create(const char *model_path, uint64_t budget_bytes, uint64_t slot_bytes,
    uint32_t slots_per_slab, const int8_t *iq2_xs_grid, uint32_t iq2_xs_grid_count,
    const int8_t *iq1_m_grid, uint32_t iq1_m_grid_count);

/* native/redmetal_ffn.h:24-31, native/redmetal_ffn.m:452-482 */
void redmetal_ffn_pool_destroy(redmetal_ffn_pool_t pool);
uint32_t redmetal_ffn_pool_capacity(redmetal_ffn_pool_t pool);
uint32_t redmetal_ffn_pool_slab_count(redmetal_ffn_pool_t pool);
uint64_t redmetal_ffn_pool_allocated_bytes(redmetal_ffn_pool_t pool);
uint64_t redmetal_ffn_pool_bytes_read(redmetal_ffn_pool_t pool);
uint64_t redmetal_ffn_pool_read_calls(redmetal_ffn_pool_t pool);
double redmetal_ffn_pool_read_ms(redmetal_ffn_pool_t pool);
int redmetal_ffn_pool_slot_inflight(redmetal_ffn_pool_t pool, uint32_t slot_id);

/* native/redmetal_ffn.h:33-43, native/redmetal_ffn.m:484-539: three preads into gate|up|down of the slot */
int redmetal_ffn_pool_load_expert(redmetal_ffn_pool_t pool, uint32_t slot_id,
    uint64_t gate_file_offset, uint64_t gate_bytes, uint64_t up_file_offset, uint64_t up_bytes,
    uint64_t down_file_offset, uint64_t down_bytes, uint64_t *bytes_read, double *elapsed_ms);

/* native/redmetal_ffn.h:45-53, native/redmetal_ffn.m:541-569: device virtual addresses of the three matrices */
int redmetal_ffn_pool_slot_addresses(redmetal_ffn_pool_t pool, uint32_t slot_id,
    uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes,
    uint64_t *gate_address, uint64_t *up_address, uint64_t *down_address);

/* native/redmetal_ffn.h:55-70, native/redmetal_ffn.m:571-706:
 * output[i] = down[output_row_start + i] . (SiLU(gate . x) * (up . x)), no router weight. */
int redmetal_ffn_pool_execute_expert(redmetal_ffn_pool_t pool, uint32_t slot_id, uint32_t ggml_type,
    uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes, uint32_t hidden_size, uint32_t ffn_size,
    uint32_t output_row_start, uint32_t output_row_count, const float *input, uint32_t input_count,
    float *output, uint32_t output_count, double *elapsed_ms);

/* No counterpart in the reference. For callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same computation as redmetal_ffn_pool_execute_expert, stream-ordered on device
 * pointers - input_dev [hidden] f32, output_dev [output_row_count] f32, `stream` a hipStream_t (NULL = the default stream), no host
 * synchronisation - and it calls no hipMalloc / hipFree. The SwiGLU activations between its two launches live in a 64 KB array
 * that is part of the library's device image (one copy per GPU, held until the process ends): ffn_size is limited to 16384
 * (larger: 0 + message). Every call on a GPU shares that GPU's array, so calls that overlap on one GPU (different streams,
 * threads or pools) race; calls on one stream are ordered. The slot must have been loaded (its slab exists); the slot is not
 * marked in flight, so the caller must not reload it before the stream has passed the call. IQ2_XS / IQ1_M experts need the
 * pool's codebooks on the device already (redmetal_ffn_pool_execute_expert on such an expert puts them there). */
int redmetal_ffn_pool_execute_expert_noalloc(redmetal_ffn_pool_t pool, uint32_t slot_id, uint32_t ggml_type,
    uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes, uint32_t hidden_size, uint32_t ffn_size,
    uint32_t output_row_start, uint32_t output_row_count, const float *input_dev, uint32_t input_count,
    float *output_dev, uint32_t output_count, void *stream);

#ifdef __cplusplus
}
#endif
