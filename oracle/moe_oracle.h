/*
 * TEST INFRASTRUCTURE - CPU oracle for the routed-expert MoE FFN path.
 *
 * A plain-C restatement of the reference's scalar, double-accumulating CPU
 * path. It exists to CHECK the HIP library and to be timed as the CPU
 * baseline. Nothing in the shipped library links, loads or calls it.
 *
 * Every function cites the reference lines it follows. Parity status:
 *   pinned by the reference's golden vectors / compiled reference / closed
 *   forms: f16 conversion, both codebooks, dequant + row_dot of IQ2_XXS,
 *   IQ3_S, Q6_K, F32 router logits, softmax top-k selection, the complete
 *   gated shared expert (rl_native_shared_cpu_execute), SiLU*up.
 *   composition only (the reference cannot run these types through its own
 *   routed-expert entry point, which rejects IQ2_XXS): orc_expert_ffn with an
 *   IQ2_XXS down projection fed double activations, orc_moe_layer. They are
 *   pinned by closed forms and by equality with the pinned pieces they
 *   compose, see tests/test_oracle_*.py.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_TYPE_F32 0u
#define ORC_TYPE_Q6_K 14u
#define ORC_TYPE_IQ2_XXS 16u
#define ORC_TYPE_IQ3_S 21u

float orc_f16_to_f32(uint16_t h);
void orc_f16_all(float *out);                  /* all 65536 bit patterns, bit-preserving (NaN payloads too) */
const uint8_t *orc_iq2xxs_grid(void);          /* [256][8] */
const uint32_t *orc_iq3s_grid(void);           /* [512] */
uint32_t orc_crc32(const void *data, size_t n);

size_t orc_block_bytes(uint32_t type);                 /* per 256 weights; 0 = unsupported */
size_t orc_row_bytes(uint32_t type, uint32_t ncols);   /* 0 = unsupported */

int orc_dequant_row(uint32_t type, const uint8_t *row, uint32_t ncols, float *out);
int orc_row_dot(uint32_t type, const uint8_t *row, const float *x, uint32_t ncols, double *out);
int orc_row_dot_d(uint32_t type, const uint8_t *row, const double *x, uint32_t ncols, double *out);
/* IQ2_XS (17, 74-byte blocks) and IQ1_M (29, 56-byte blocks): the reference's current routed-expert formats. Their
 * codebooks are arguments, as in the reference (512 x 8 resp. 2048 x 8 int8 values, native/redlite_native_tables.c).
 * Dequantised weights (exact in f32) and the double-accumulated row dot of native/redlite_native_reference.c:116-172. */
int orc_dequant_row_grid(uint32_t type, const uint8_t *row, uint32_t ncols, const int8_t *grid, float *out);
/* keep copies of the IQ2_XS (512 x 8) / IQ1_M (2048 x 8) codebooks for the functions without a grid argument; NULL: unchanged */
void orc_set_codebooks(const int8_t *iq2_xs, const int8_t *iq1_m);
int orc_row_dot_grid(uint32_t type, const uint8_t *row, const float *x, uint32_t ncols, const int8_t *grid, double *out);
/* single-expert FFN where either side may be a codebook format (17 / 29); other types as orc_expert_ffn */
int orc_expert_ffn_grid(uint32_t gate_up_type, uint32_t down_type, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                        uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count, const float *x,
                        const int8_t *xs_grid, const int8_t *m_grid, double *out);

/* out[r] = (float) row_dot(W[row_start + r], x); rows split over `threads` pthreads like the reference's matvec */
int orc_matvec(uint32_t type, const uint8_t *w, uint32_t ncols, uint32_t row_start, uint32_t row_count,
               const float *x, float *out, int threads);

void orc_rmsnorm(const float *x, const float *w, uint32_t n, float eps, float *out);

int orc_router_logits(uint32_t type, const uint8_t *w, uint32_t hidden, uint32_t experts, const float *x, float *logits);
int orc_router_select(const float *logits, uint32_t experts, uint32_t top_k, uint32_t *ids, float *weights, float *probs);

double orc_silu_mul(double gate, double up);

/* one routed expert, no router weight: out[i] = down[row_start+i] . (silu(gate.x) * (up.x)), activations kept in double */
int orc_expert_ffn(uint32_t gate_up_type, uint32_t down_type,
                   const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                   uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count,
                   const float *x, double *out);

/* out[r] = sum_k (double)weights[k] * expert_k[r], experts in selection order. experts are addressed through
 * three base pointers and per-expert strides (bytes). */
int orc_routed_topk(uint32_t gate_up_type, uint32_t down_type,
                    const uint8_t *gate_base, const uint8_t *up_base, const uint8_t *down_base,
                    size_t gate_stride, size_t up_stride, size_t down_stride,
                    const uint32_t *ids, const float *weights, uint32_t top_k,
                    uint32_t hidden, uint32_t ffn, const float *x, double *out);

/* engine-style shared expert: float hand-offs, exp() in double. out_sh[hidden] floats, *scalar = sigmoid(gate_inp . x) */
int orc_shared_expert(uint32_t gate_up_type, uint32_t down_type,
                      const uint8_t *gate, const uint8_t *up, const uint8_t *down, const float *gate_inp,
                      uint32_t hidden, uint32_t ffn, const float *x, float *out_sh, double *scalar, int threads);

/* stand-alone shared expert variant (expf in float, double output already multiplied by the scalar gate) */
int orc_shared_expert_standalone(uint32_t gate_up_type, uint32_t down_type,
                      const uint8_t *gate, const uint8_t *up, const uint8_t *down, const float *gate_inp,
                      uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count,
                      const float *x, double *out, double *scalar);

typedef struct {
    uint32_t hidden, ffn, n_expert, top_k;
    uint32_t router_type;                  /* 0 or 14 */
    uint32_t gate_up_type, down_type;      /* routed experts */
    uint32_t sh_gate_up_type, sh_down_type;
    const uint8_t *router;                 /* [n_expert] rows of hidden weights */
    const uint8_t *gate, *up, *down;       /* expert-major, contiguous experts */
    const uint8_t *sh_gate, *sh_up, *sh_down;
    const float *sh_gate_inp;              /* [hidden] */
} orc_layer;

/* complete layer for one token: logits -> select -> routed -> shared -> combine. ids/weights/logits may be NULL. */
int orc_moe_layer(const orc_layer *L, const float *x, float *out, uint32_t *ids, float *weights, float *logits, int threads);

/* token grouping: ids/weights are [ntok][top_k]. Outputs: uid[U] (first-appearance order), expert_start[U+1],
 * pair_token[P], pair_weight[P], tok_pair[P], P = ntok*top_k. Returns U, or -1 on bad arguments. */
int orc_group_pairs(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t n_expert,
                    uint32_t *uid, uint32_t *expert_start, uint32_t *pair_token, float *pair_weight, uint32_t *tok_pair);

/* batched layer (ntok tokens) = orc_moe_layer per token; here for the CPU baseline of small batches */
int orc_moe_layer_batch(const orc_layer *L, const float *x, uint32_t ntok, float *out, uint32_t *ids, float *weights, int threads);

#ifdef __cplusplus
}
#endif
