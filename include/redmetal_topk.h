/*
 * Resident top-k expert pool - C ABI of libredmetal_hip.so (MI355X / gfx950).
 *
 * Replaces the pool the reference declares in native/redmetal_topk.h:11-245 and implements in
 * native/redmetal_topk.m:1125-2062. Names, argument order and meaning, the return convention (1 = success, 0 = failure
 * with a message through redmetal_topk_last_error(), thread-local) and the slot layout gate|up|down are kept, so an
 * engine written against the reference binds this library unchanged. What a Metal object was there is a HIP object here,
 * passed through the same `void *` parameter:
 *     id<MTLCommandBuffer> / id<MTLComputeCommandEncoder>   ->  hipStream_t (NULL = the default stream)
 *     id<MTLBuffer> + byte offset                           ->  device pointer + byte offset
 * "Encode" therefore means: enqueue on that stream, no host synchronisation. Host arrays handed to an encode call (slot
 * ids, weights, pair lists) are copied before the call returns.
 *
 * Differences, all additive: ggml_type accepts IQ2_XXS (16), IQ3_S (21) and Q6_K (14) beside the reference's IQ2_XS (17) /
 * IQ1_M (29) and the two-type word gate_up | down << 8 (native/redmetal_topk.m:41-50). The process holds one device copy of
 * the IQ2_XS / IQ1_M codebooks: a pool binds to their content when it first runs such an expert, and a pool with different
 * tables fails with a message while other users of the bound tables are alive.
 * The activations between the launches of a call live in buffers of the pool (as in the reference): calls on one stream are
 * ordered; calls on different streams that overlap race.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *redmetal_topk_pool_t;

/* experts per encoded plan, native/redmetal_topk.m:54 */
#define REDMETAL_TOPK_MAX 512u
/* native/redmetal_topk.h:25 */
#define RL_TOPK_MAX_CLASSES 8u

/* native/redmetal_topk.h:11-12, native/redmetal_topk.m:1125-1128 */
uint32_t redmetal_topk_abi_version(void);
const char *redmetal_topk_last_error(void);

/* native/redmetal_topk.h:14-22, native/redmetal_topk.m:1130-1151. slot size rounded up to 4096; capacity = budget / slot
 * size; slabs of slots_per_slab (0 = 64) slots are allocated in HBM on first use. Both codebooks are required
 * (512 x 8 and 2048 x 8 values). */
redmetal_topk_pool_t redmetal_topk_pool_create(const char *model_path, uint64_t budget_bytes, uint64_t slot_bytes,
    uint32_t slots_per_slab, const int8_t *iq2_xs_grid, uint32_t iq2_xs_grid_count,
    const int8_t *iq1_m_grid, uint32_t iq1_m_grid_count);
void redmetal_topk_pool_destroy(redmetal_topk_pool_t pool);

/* native/redmetal_topk.h:24-26, native/redmetal_topk.m:937-972: slot size classes (slots of class c follow those of class
 * c - 1), only before any slab exists and within the budget; capacity becomes the sum. */
int redmetal_topk_pool_set_classes(redmetal_topk_pool_t pool, uint32_t n, const uint64_t *slot_bytes, const uint32_t *capacity);

/* native/redmetal_topk.h:27-35, native/redmetal_topk.m:1171-1199 */
uint32_t redmetal_topk_pool_capacity(redmetal_topk_pool_t pool);
uint32_t redmetal_topk_pool_slab_count(redmetal_topk_pool_t pool);
uint64_t redmetal_topk_pool_allocated_bytes(redmetal_topk_pool_t pool);
uint64_t redmetal_topk_pool_bytes_read(redmetal_topk_pool_t pool);
uint64_t redmetal_topk_pool_read_calls(redmetal_topk_pool_t pool);
double redmetal_topk_pool_read_ms(redmetal_topk_pool_t pool);
uint32_t redmetal_topk_pool_slot_generation(redmetal_topk_pool_t pool, uint32_t slot_id);      /* loads ever written into the slot */
int redmetal_topk_pool_slot_inflight(redmetal_topk_pool_t pool, uint32_t slot_id);

/* native/redmetal_topk.h:37-47, native/redmetal_topk.m:1201-1259: three preads into gate|up|down of the slot (through pinned
 * host memory into HBM); refuses a slot that is in flight; counts the generation. */
int redmetal_topk_pool_load_expert(redmetal_topk_pool_t pool, uint32_t slot_id,
    uint64_t gate_file_offset, uint64_t gate_bytes, uint64_t up_file_offset, uint64_t up_bytes,
    uint64_t down_file_offset, uint64_t down_bytes, uint64_t *bytes_read, double *elapsed_ms);

/* native/redmetal_topk.h:49-57, native/redmetal_topk.m:1261-1289: device virtual addresses of the three matrices */
int redmetal_topk_pool_slot_addresses(redmetal_topk_pool_t pool, uint32_t slot_id,
    uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes,
    uint64_t *gate_address, uint64_t *up_address, uint64_t *down_address);

/* native/redmetal_topk.h:59-76, native/redmetal_topk.m:1291-1336 (validation) and :1417-1472:
 * output[i] = sum_k router_weights[k] * (down_k[output_row_start + i] . (SiLU(gate_k . x) * (up_k . x))), k in list order.
 * Host pointers, synchronous. Slot ids must be distinct and below the capacity; the byte counts must be those of the
 * shapes and types. */
int redmetal_topk_pool_execute(redmetal_topk_pool_t pool, const uint32_t *slot_ids,
    const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes,
    const float *router_weights, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
    uint32_t output_row_start, uint32_t output_row_count, const float *input, uint32_t input_count,
    float *output, uint32_t output_count, double *elapsed_ms);

/* native/redmetal_topk.h:78-102, native/redmetal_topk.m:2018-2056 (and :1338-1415): the same three launches enqueued on
 * `stream`, input vector at input_dev + input_offset bytes, output rows at output_dev + output_offset bytes. Marks the
 * slots in flight; call redmetal_topk_pool_release once the stream has passed the work. */
int redmetal_topk_pool_encode(redmetal_topk_pool_t pool, void *stream, const uint32_t *slot_ids,
    const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes,
    const float *router_weights, uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size,
    uint32_t output_row_start, uint32_t output_row_count, void *input_dev, uint64_t input_offset,
    void *output_dev, uint64_t output_offset);
/* native/redmetal_topk.h:104, native/redmetal_topk.m:2058-2062 */
void redmetal_topk_pool_release(redmetal_topk_pool_t pool, const uint32_t *slot_ids, uint32_t top_k);

/* native/redmetal_topk.h:106-120, native/redmetal_topk.m:1714-1775. The residency table is uint64_t[layers][experts] in
 * device memory (0 = not resident) that a routing kernel can read; _set / _clear update it with a small synchronous copy.
 * redmetal_topk_pool_residency_table returns its device pointer. allocate_all creates every slab now. There is no
 * residency-set object on this platform: slab_residency_set returns NULL (as the reference does before macOS 15) and
 * use_all_slabs does nothing (device memory needs no per-launch declaration). */
int redmetal_topk_pool_residency_table_init(redmetal_topk_pool_t pool, uint32_t layers, uint32_t experts);
void *redmetal_topk_pool_residency_table(redmetal_topk_pool_t pool);
int redmetal_topk_pool_residency_set(redmetal_topk_pool_t pool, uint32_t layer, uint32_t expert, uint32_t slot_id);
void redmetal_topk_pool_residency_clear(redmetal_topk_pool_t pool, uint32_t layer, uint32_t expert);
void *redmetal_topk_pool_slab_residency_set(redmetal_topk_pool_t pool);
int redmetal_topk_pool_allocate_all(redmetal_topk_pool_t pool);
void redmetal_topk_pool_use_all_slabs(redmetal_topk_pool_t pool, void *stream);

/* native/redmetal_topk.h:122-144 and :175-190, native/redmetal_topk.m:1777-1856, :1858-1943, :1979-1995: one token, the slot
 * table (uint64_t slot base addresses, top_k entries, e.g. rows of the residency table gathered by a routing kernel) and the
 * router weights (float[top_k]) read from device memory, so no host round trip is needed. No in-flight marking. gate_bytes /
 * up_bytes place the up and down matrices inside a slot. With output_dev NULL the weighted sum is not enqueued and the
 * per-expert down outputs stay in redmetal_topk_pool_tmp_buffer() as tmp[e * hidden_size + r]. encode_device and
 * encode_device_into differ in the reference only in the Metal object they append to; here both take the stream. */
int redmetal_topk_pool_encode_device(redmetal_topk_pool_t pool, void *stream,
    void *slot_table_dev, uint64_t slot_table_offset, void *weight_dev, uint64_t weight_offset,
    uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint64_t gate_bytes, uint64_t up_bytes,
    void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset);
int redmetal_topk_pool_encode_device_into(redmetal_topk_pool_t pool, void *stream,
    void *slot_table_dev, uint64_t slot_table_offset, void *weight_dev, uint64_t weight_offset,
    uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint64_t gate_bytes, uint64_t up_bytes,
    void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset);
/* Device pointer; NULL before the first single-token encode. Sized REDMETAL_TOPK_MAX * hidden_size floats by the single-token
 * encodes only: the pointer stays valid until an encode with a larger hidden_size (or ffn_size) than any before it; the batched /
 * mapped forms use buffers of their own and never move it. */
void *redmetal_topk_pool_tmp_buffer(redmetal_topk_pool_t pool);

/* native/redmetal_topk.h:156-161, native/redmetal_topk.m:1997-2016 (kernel :209-252): as encode_device_into, but the experts
 * from index x_split on read the second input vector (two-row verify). */
int redmetal_topk_pool_encode_device_into2(redmetal_topk_pool_t pool, void *stream,
    void *slot_table_dev, uint64_t slot_table_offset, void *weight_dev, uint64_t weight_offset,
    uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint64_t gate_bytes, uint64_t up_bytes,
    void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset,
    void *input1_dev, uint64_t input1_offset, uint32_t x_split);

/* native/redmetal_topk.h:162-169, native/redmetal_topk.m:1945-1977 (kernel :254-281): gate/up, down, then the MoE tail in the
 * last launch: v = resid[r] + (sum_k w[k] * down_k[r] . act_k + shared[r] * scalar[0]) written to x[r] and to layer_out[r]
 * (at layer_out_offset bytes). Returns -1, nothing enqueued, for more than 64 experts (the reference's limit; its second
 * condition, eight lanes per down row, is a property of its kernel and does not apply here). */
int redmetal_topk_pool_encode_device_tail(redmetal_topk_pool_t pool, void *stream,
    void *slot_table_dev, uint64_t slot_table_offset, void *weight_dev, uint64_t weight_offset,
    uint32_t top_k, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint64_t gate_bytes, uint64_t up_bytes,
    void *input_dev, uint64_t input_offset, void *resid_dev, void *shared_dev, void *scalar_dev, void *x_dev,
    void *layer_out_dev, uint64_t layer_out_offset);

/* Batched prefill, native/redmetal_topk.h:192-245, native/redmetal_topk.m:1474-1602 and :1664-1712: n_expert distinct experts
 * (slots) serve n_pairs = ntok * top_k (expert, token) pairs sorted by expert (expert_start[n_expert + 1] prefix sums;
 * pair_token / pair_weight per pair; tok_pair[ntok * top_k] lists each token's pairs in router selection order; all four are
 * host arrays). Input rows are hidden_size floats per token at input_dev + input_offset (token index = pair_token), output
 * rows likewise for tokens tok_first .. tok_first + ntok - 1. Every expert's weights are decoded once per eight of its
 * pairs. Marks the slots in flight; release with redmetal_topk_pool_release(slot_ids, n_expert). */
int redmetal_topk_pool_encode_batched(redmetal_topk_pool_t pool, void *stream, const uint32_t *slot_ids,
    const uint64_t *gate_bytes, const uint64_t *up_bytes, const uint64_t *down_bytes, uint32_t n_expert,
    uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint32_t tok_first, uint32_t ntok, uint32_t top_k,
    uint32_t n_pairs, const uint32_t *pair_token, const float *pair_weight, const uint32_t *expert_start,
    const uint32_t *tok_pair, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset);

/* native/redmetal_topk.h:199-232, native/redmetal_topk.m:1604-1662: the same pair layout on experts read in place from three
 * device ranges holding whole tensors (expert e of the gate tensor at gate_addr0 + e * gate_bytes, and so on); the first
 * of each pair of arguments (the Metal buffer the address lies in) is not needed here and may be NULL. No slots, no
 * in-flight marking. */
int redmetal_topk_pool_encode_mapped(redmetal_topk_pool_t pool, void *stream,
    void *gate_buffer, uint64_t gate_addr0, void *up_buffer, uint64_t up_addr0, void *down_buffer, uint64_t down_addr0,
    uint64_t gate_bytes, uint64_t up_bytes, uint64_t down_bytes, const uint32_t *expert_ids, uint32_t n_expert,
    uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint32_t tok_first, uint32_t ntok, uint32_t top_k,
    uint32_t n_pairs, const uint32_t *pair_token, const float *pair_weight, const uint32_t *expert_start,
    const uint32_t *tok_pair, void *input_dev, uint64_t input_offset, void *output_dev, uint64_t output_offset);

/* No counterpart in the reference. Opt-in, after redmetal_topk_pool_set_classes (if used) and before the first slab exists (no load,
 * no slot_addresses, no allocate_all yet): experts of one declared shape - every matrix IQ2_XXS (type word 16) with hidden_size in
 * {512, 1024, 2048, 4096}, or IQ2_XXS gate / up with IQ3_S down (16 | 21 << 8), every matrix IQ2_XS (17) or every matrix IQ1_M (29, the
 * last two decoded through the pool's codebooks) with hidden_size in {512, 1024, 2048}; ffn_size a multiple of 256 up to 1024 - also
 * keep, behind the raw bytes of their slot, a copy in the
 * layout this library's fused kernels read (packed gate | up streams, column-sliced down matrix), written by
 * redmetal_topk_pool_load_expert. The single-token calls (encode, execute, encode_device, _into, _into2 with an output, _tail) of that
 * shape with whole output rows and top_k <= 64 then run as two launches on those copies instead of three on the raw rows; every other
 * call runs as before, and redmetal_topk_pool_slot_addresses keeps returning the raw bytes. The copies count against the budget: a
 * slot class that holds such experts grows to about twice the expert's bytes - the raw bytes rounded up to 256, then the copy: 8 bytes
 * per 32 weights + 2 per 256 (IQ2_XS 9 per 32, IQ3_S down 16 per 32), the whole rounded up to 4096 - (a single-class pool's capacity shrinks accordingly; with
 * classes set, the call fails when they no longer fit). With the device-driven forms the slot table must hold addresses of this
 * pool's slots loaded with experts of the declared shape. flags: REDHIP_TOPK_FAST_TILES (hidden_size <= 2048 and ffn_size <= 512)
 * adds a third copy per slot, tile-major as this library's prefill kernels read it (the slot class grows to three times the expert's
 * bytes); redmetal_topk_pool_encode_batched of that shape then runs on those kernels - tiles of up to 32 pairs per expert on the
 * matrix units - when every slot it names holds its copies; 0: none. Returns 1, or 0 with redmetal_topk_last_error(). */
#define REDHIP_TOPK_FAST_TILES 1u
int redhip_topk_pool_enable_fast_path(redmetal_topk_pool_t pool, uint32_t ggml_type, uint32_t hidden_size, uint32_t ffn_size, uint32_t flags);

#ifdef __cplusplus
}
#endif
