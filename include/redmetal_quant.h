/*
 * One-shot quantised GEMV - C ABI of libredmetal_hip.so (MI355X / gfx950).
 *
 * Replaces native/redmetal_quant.h:9-28 (implementation native/redmetal_quant.m:146-303): reads a row-major
 * quantised matrix from a file and returns rows [row_start, row_start + row_count) of W . x. Same signature
 * and error convention (1/0, redmetal_quant_last_error(), thread-local, cleared on entry).
 * ggml_type: the reference's IQ2_XS (17) / IQ1_M (29), decoded through the caller's `grid` (512 x 8 resp. 2048 x 8 int8 values, exact
 * count required, as native/redmetal_quant.m:160-170), plus F32 (0), Q6_K (14), IQ2_XXS (16), IQ3_S (21), for which `grid` may be
 * NULL / 0: these formats carry built-in codebooks.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

uint32_t redmetal_quant_abi_version(void);      /* native/redmetal_quant.h:9 */
const char *redmetal_quant_last_error(void);    /* native/redmetal_quant.h:10 */

/* native/redmetal_quant.h:12-28 */
int redmetal_quant_rows(const char *model_path, uint64_t matrix_file_offset, uint64_t matrix_bytes,
    uint32_t ggml_type, uint32_t ncols, uint32_t nrows, uint32_t row_start, uint32_t row_count,
    const float *input, uint32_t input_count, const int8_t *grid, uint32_t grid_count,
    float *output, uint32_t output_count, double *io_ms, double *gpu_ms);

#ifdef __cplusplus
}
#endif
