/*
 * Golden-vector generator. Runs ONLY in the build container, where the reference checkout exists:
 * it calls the reference's own portable C (compiled unchanged into oracle/_ref/libref.so by
 * oracle/Makefile) on small seeded inputs and writes inputs + outputs to JSON fixtures. The
 * fixtures are data; nothing of the reference's source text is stored.
 *
 *   make -C oracle ref && sh tests/golden/make_golden.sh
 *
 * Reference entry points exercised (native/...):
 *   rl_quant_dequant_row / rl_quant_row_dot      redlite_native_quant_cpu.c:155-280   types 0, 14, 16, 21
 *   rl_iq3_row_dot_d                             redlite_native_iq3.c:135-148         type 21, double input
 *   rl_native_router_select_softmax_topk         redlite_native_router_exec.c:102-184
 *   rl_native_router_cpu_f32                     redlite_native_router_exec.c:37-100
 *   rl_native_shared_cpu_execute                 redlite_native_shared_exec.c:228-314
 *   rl_quant_f16_to_f32                          redlite_native_quant_cpu.c:20-38
 */
#define _POSIX_C_SOURCE 200809L
#include "redlite_native_iq2_xxs.h"
#include "redlite_native_iq3.h"
#include "redlite_native_quant_cpu.h"
#include "redlite_native_router_exec.h"
#include "redlite_native_shared_exec.h"

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static uint64_t g_state;
static uint32_t rnd32(void) {              /* splitmix64, upper half */
    uint64_t z = (g_state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return (uint32_t)((z ^ (z >> 31)) >> 32);
}
static float rnd_unit(void) { return (float)(rnd32() >> 8) * (1.0f / 16777216.0f); }
static float rnd_normal(void) {
    float u1 = rnd_unit(), u2 = rnd_unit();
    if (u1 < 1e-7f) u1 = 1e-7f;
    return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
}

static uint32_t crc32_bytes(const void *data, size_t n) {
    const uint8_t *p = (const uint8_t *)data;
    uint32_t c = 0xffffffffu;
    for (size_t i = 0; i < n; ++i) {
        c ^= p[i];
        for (int k = 0; k < 8; ++k) c = (c >> 1) ^ (0xedb88320u & (0u - (c & 1u)));
    }
    return c ^ 0xffffffffu;
}

static void hex(FILE *f, const char *key, const void *data, size_t n, int last) {
    const uint8_t *p = (const uint8_t *)data;
    fprintf(f, "\"%s\": \"", key);
    for (size_t i = 0; i < n; ++i) fprintf(f, "%02x", p[i]);
    fprintf(f, "\"%s", last ? "" : ", ");
}

/* f16 bit pattern with value in [lo, hi): built from the float by truncation (any valid half is fine) */
static uint16_t half_bits_from_float(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    const int32_t e = (int32_t)((b >> 23) & 255u) - 127 + 15;
    if (e <= 0) return 0;
    return (uint16_t)(((b >> 16) & 0x8000u) | ((uint32_t)e << 10) | ((b & 0x7fffffu) >> 13));
}

static size_t block_bytes(uint32_t t) { return t == 14u ? 210u : t == 16u ? 66u : 110u; }
static size_t d_offset(uint32_t t) { return t == 14u ? 208u : 0u; }

enum { FILL_RANDOM = 0, FILL_ZERO, FILL_ONES, FILL_SUBNORMAL_D, FILL_ZERO_D, FILL_NEG_D };

static void fill_row(uint32_t type, uint32_t ncols, int mode, uint8_t *row) {
    const size_t bb = block_bytes(type);
    for (uint32_t b = 0; b < ncols / 256u; ++b) {
        uint8_t *bp = row + b * bb;
        for (size_t i = 0; i < bb; ++i)
            bp[i] = mode == FILL_ZERO ? 0u : mode == FILL_ONES ? 0xffu : (uint8_t)rnd32();
        uint16_t d = half_bits_from_float(1e-3f + rnd_unit() * (2e-2f - 1e-3f));
        if (mode == FILL_SUBNORMAL_D) d = (uint16_t)(1u + (rnd32() % 1023u));
        if (mode == FILL_ZERO_D) d = 0u;
        if (mode == FILL_NEG_D) d |= 0x8000u;
        if (mode == FILL_ZERO || mode == FILL_ONES) d = 0x3c00u;
        bp[d_offset(type)] = (uint8_t)(d & 255u);
        bp[d_offset(type) + 1u] = (uint8_t)(d >> 8);
    }
}

static int rows_fixture(const char *path, const uint8_t *grid) {
    FILE *f = fopen(path, "w");
    if (!f) { perror(path); return 0; }
    fprintf(f, "{\"about\": \"reference rl_quant_dequant_row / rl_quant_row_dot / rl_iq3_row_dot_d on seeded rows; "
               "floats and doubles as little-endian hex\",\n \"cases\": [\n");
    const uint32_t types[3] = {16u, 21u, 14u};
    const uint32_t widths[3] = {256u, 512u, 2048u};
    const int modes[6] = {FILL_RANDOM, FILL_ZERO, FILL_ONES, FILL_SUBNORMAL_D, FILL_ZERO_D, FILL_NEG_D};
    int first = 1;
    for (int ti = 0; ti < 3; ++ti) for (int wi = 0; wi < 3; ++wi) for (int mi = 0; mi < 6; ++mi) {
        const uint32_t type = types[ti], ncols = widths[wi];
        if (mi > 0 && wi != 1) continue;               /* edge fills only at one width */
        const int reps = mi == 0 ? 3 : 1;
        for (int rep = 0; rep < reps; ++rep) {
            const size_t rb = block_bytes(type) * (ncols / 256u);
            uint8_t *row = (uint8_t *)malloc(rb);
            float *x = (float *)malloc(sizeof(float) * ncols);
            double *xd = (double *)malloc(sizeof(double) * ncols);
            float *w = (float *)malloc(sizeof(float) * ncols);
            fill_row(type, ncols, modes[mi], row);
            for (uint32_t i = 0; i < ncols; ++i) { x[i] = rnd_normal(); xd[i] = (double)rnd_normal() * 1.000000123; }
            double dot = 0.0, dot_d = 0.0;
            if (!rl_quant_dequant_row(type, row, ncols, grid, w) || !rl_quant_row_dot(type, row, x, ncols, grid, &dot)) {
                fprintf(stderr, "reference rejected type %u\n", type); return 0;
            }
            const int has_d = type == 21u && rl_iq3_row_dot_d(type, row, xd, ncols, &dot_d);
            fprintf(f, "%s  {\"type\": %u, \"ncols\": %u, \"fill\": %d, ", first ? "" : ",\n", type, ncols, modes[mi]);
            hex(f, "row", row, rb, 0);
            hex(f, "x", x, sizeof(float) * ncols, 0);
            hex(f, "dequant", w, sizeof(float) * ncols, 0);
            fprintf(f, "\"dequant_crc32\": \"%08x\", ", crc32_bytes(w, sizeof(float) * ncols));
            hex(f, "dot", &dot, 8, !has_d);
            if (has_d) { hex(f, "xd", xd, sizeof(double) * ncols, 0); hex(f, "dot_d", &dot_d, 8, 1); }
            fprintf(f, "}");
            first = 0;
            free(row); free(x); free(xd); free(w);
        }
    }
    /* F32 rows (type 0) through the same entry point */
    for (int rep = 0; rep < 2; ++rep) {
        const uint32_t ncols = 2048u;
        float *wrow = (float *)malloc(sizeof(float) * ncols), *x = (float *)malloc(sizeof(float) * ncols);
        for (uint32_t i = 0; i < ncols; ++i) { wrow[i] = 0.02f * rnd_normal(); x[i] = rnd_normal(); }
        double dot = 0.0;
        rl_quant_row_dot(0u, (const uint8_t *)wrow, x, ncols, NULL, &dot);
        fprintf(f, ",\n  {\"type\": 0, \"ncols\": %u, \"fill\": 0, ", ncols);
        hex(f, "row", wrow, sizeof(float) * ncols, 0);
        hex(f, "x", x, sizeof(float) * ncols, 0);
        hex(f, "dot", &dot, 8, 1);
        fprintf(f, "}");
        free(wrow); free(x);
    }
    fprintf(f, "\n ]}\n");
    fclose(f);
    return 1;
}

static int router_fixture(const char *path) {
    FILE *f = fopen(path, "w");
    if (!f) { perror(path); return 0; }
    fprintf(f, "{\"about\": \"reference rl_native_router_select_softmax_topk; floats as little-endian hex\",\n \"cases\": [\n");
    int first = 1;
    for (int c = 0; c < 12; ++c) {
        const uint32_t E = c < 8 ? 512u : (c == 8 ? 4u : c == 9 ? 16u : 64u), K = c < 8 ? 10u : (c == 8 ? 2u : 4u);
        float *l = (float *)malloc(sizeof(float) * E), *p = (float *)malloc(sizeof(float) * E);
        for (uint32_t i = 0; i < E; ++i) l[i] = rnd_normal() * (c == 1 ? 8.0f : 1.0f);
        if (c == 2) for (uint32_t i = 0; i < E; ++i) l[i] = (float)((i * 7u) % 5u);              /* heavy exact ties */
        if (c == 3) for (uint32_t i = 0; i < E; ++i) l[i] = 0.25f;                                /* all equal */
        if (c == 4) for (uint32_t i = 0; i < 32u; ++i) l[(i * 37u) % E] += 2.0f;                  /* hot experts */
        if (c == 5) for (uint32_t i = 0; i < E; ++i) l[i] = -80.0f + (i == 77u ? 90.0f : 0.0f) + 1e-3f * (float)(i % 3u); /* underflow tail */
        if (c == 6) { l[100] = l[7] = l[300] = 3.5f; l[8] = nextafterf(3.5f, 4.0f); }             /* near and exact ties at the top */
        if (c == 7) for (uint32_t i = 0; i < E; ++i) l[i] = (float)(sin(0.37 * i) * 3.0) + (i % 7u == 0u ? 0.5f : 0.0f);
        uint32_t ids[16];
        float w[16];
        char err[128];
        if (!rl_native_router_select_softmax_topk(l, E, K, ids, w, p, err, sizeof(err))) { fprintf(stderr, "select: %s\n", err); return 0; }
        fprintf(f, "%s  {\"experts\": %u, \"top_k\": %u, ", first ? "" : ",\n", E, K);
        hex(f, "logits", l, sizeof(float) * E, 0);
        fprintf(f, "\"ids\": [");
        for (uint32_t k = 0; k < K; ++k) fprintf(f, "%u%s", ids[k], k + 1 < K ? ", " : "");
        fprintf(f, "], ");
        hex(f, "weights", w, sizeof(float) * K, 0);
        hex(f, "probs", p, sizeof(float) * E, 1);
        fprintf(f, "}");
        first = 0;
        free(l); free(p);
    }
    fprintf(f, "\n ]}\n");
    fclose(f);
    return 1;
}

/* complete gated shared expert and F32 router logits through the reference's file-based entry points */
static int shared_fixture(const char *path, const char *tmp_path) {
    FILE *f = fopen(path, "w");
    if (!f) { perror(path); return 0; }
    fprintf(f, "{\"about\": \"reference rl_native_shared_cpu_execute and rl_native_router_cpu_f32 on a raw synthetic file; "
               "file layout: gate_inp f32[hidden] | gate | up | down | router f32[experts][hidden]\",\n \"cases\": [\n");
    const uint32_t H = 512u, F = 256u, E = 16u;
    int first = 1;
    for (int c = 0; c < 3; ++c) {
        const uint32_t gu = c == 1 ? 14u : 16u, dn = c == 0 ? 16u : 14u;
        const size_t grb = block_bytes(gu) * (H / 256u), drb = block_bytes(dn) * (F / 256u);
        const size_t n_inp = 4u * H, n_g = F * grb, n_d = H * drb, n_r = 4u * (size_t)E * H;
        const size_t total = n_inp + 2u * n_g + n_d + n_r;
        uint8_t *file = (uint8_t *)malloc(total);
        float *gi = (float *)file;
        for (uint32_t i = 0; i < H; ++i) gi[i] = 0.02f * rnd_normal();
        for (uint32_t r = 0; r < F; ++r) { fill_row(gu, H, FILL_RANDOM, file + n_inp + r * grb); fill_row(gu, H, FILL_RANDOM, file + n_inp + n_g + r * grb); }
        for (uint32_t r = 0; r < H; ++r) fill_row(dn, F, FILL_RANDOM, file + n_inp + 2u * n_g + r * drb);
        float *rw = (float *)(file + n_inp + 2u * n_g + n_d);
        for (uint32_t i = 0; i < E * H; ++i) rw[i] = 0.02f * rnd_normal();
        FILE *t = fopen(tmp_path, "wb");
        if (!t || fwrite(file, 1, total, t) != total) { perror(tmp_path); return 0; }
        fclose(t);
        float x[512];
        double ss = 0.0;
        for (uint32_t i = 0; i < H; ++i) { x[i] = rnd_normal(); ss += (double)x[i] * x[i]; }
        for (uint32_t i = 0; i < H; ++i) x[i] = (float)(x[i] / sqrt(ss / H + 1e-6));
        rl_shared_tensor_info ti[4];
        memset(ti, 0, sizeof(ti));
        for (int k = 0; k < 4; ++k) { ti[k].layer = 0; ti[k].kind = (rl_shared_kind)k; }
        ti[0].ggml_type = 0u; ti[0].n_dims = 1u; ti[0].shape[0] = H; ti[0].tensor_offset = 0; ti[0].tensor_span_bytes = n_inp;
        ti[1].ggml_type = gu; ti[1].n_dims = 2u; ti[1].shape[0] = H; ti[1].shape[1] = F; ti[1].tensor_offset = n_inp; ti[1].tensor_span_bytes = n_g;
        ti[2] = ti[1]; ti[2].kind = RL_SHARED_UP; ti[2].tensor_offset = n_inp + n_g;
        ti[3].ggml_type = dn; ti[3].n_dims = 2u; ti[3].shape[0] = F; ti[3].shape[1] = H; ti[3].tensor_offset = n_inp + 2u * n_g; ti[3].tensor_span_bytes = n_d;
        double out[512];
        rl_native_shared_telemetry tel;
        char err[256] = {0};
        if (!rl_native_shared_cpu_execute(tmp_path, ti, x, H, 0u, H, out, H, &tel, err, sizeof(err))) { fprintf(stderr, "shared: %s\n", err); return 0; }
        rl_router_tensor_info ri;
        memset(&ri, 0, sizeof(ri));
        ri.ggml_type = 0u; ri.n_dims = 2u; ri.shape[0] = H; ri.shape[1] = E; ri.tensor_offset = n_inp + 2u * n_g + n_d; ri.tensor_span_bytes = n_r;
        float logits[16];
        if (!rl_native_router_cpu_f32(tmp_path, &ri, x, H, logits, E, NULL, err, sizeof(err))) { fprintf(stderr, "router: %s\n", err); return 0; }
        fprintf(f, "%s  {\"hidden\": %u, \"ffn\": %u, \"experts\": %u, \"gate_up_type\": %u, \"down_type\": %u, ", first ? "" : ",\n", H, F, E, gu, dn);
        hex(f, "file", file, total, 0);
        hex(f, "x", x, sizeof(x), 0);
        hex(f, "out", out, sizeof(out), 0);
        hex(f, "scalar_gate", &tel.scalar_gate, 8, 0);
        hex(f, "router_logits", logits, sizeof(logits), 1);
        fprintf(f, "}");
        first = 0;
        free(file);
    }
    fprintf(f, "\n ]}\n");
    fclose(f);
    remove(tmp_path);
    return 1;
}

static int f16_fixture(const char *path) {
    FILE *f = fopen(path, "w");
    if (!f) { perror(path); return 0; }
    float *all = (float *)malloc(sizeof(float) * 65536u);
    for (uint32_t h = 0; h < 65536u; ++h) all[h] = rl_quant_f16_to_f32((uint16_t)h);
    /* NaN payloads are included: the conversion is a pure bit map */
    fprintf(f, "{\"about\": \"reference rl_quant_f16_to_f32 over all 65536 bit patterns\", \"crc32_of_f32_le\": \"%08x\", "
               "\"spot\": {\"0001\": \"%08x\", \"03ff\": \"%08x\", \"0400\": \"%08x\", \"3c00\": \"%08x\", \"7bff\": \"%08x\", \"fc00\": \"%08x\", \"8001\": \"%08x\"}}\n",
            crc32_bytes(all, sizeof(float) * 65536u), *(uint32_t *)&all[1], *(uint32_t *)&all[0x3ff], *(uint32_t *)&all[0x400],
            *(uint32_t *)&all[0x3c00], *(uint32_t *)&all[0x7bff], *(uint32_t *)&all[0xfc00], *(uint32_t *)&all[0x8001]);
    fclose(f);
    free(all);
    return 1;
}

int main(int argc, char **argv) {
    if (argc != 2) { fprintf(stderr, "usage: %s <output dir>\n", argv[0]); return 2; }
    uint8_t grid[RL_IQ2_XXS_GRID_COUNT];
    char err[256];
    if (!rl_native_iq2_xxs_build_grid(grid, err, sizeof(err))) { fprintf(stderr, "%s\n", err); return 1; }
    if (!rl_quant_selftest(err, sizeof(err)) || !rl_iq3_selftest(err, sizeof(err))) { fprintf(stderr, "reference selftest: %s\n", err); return 1; }
    char p[512], t[512];
    g_state = 0x5eed0001ull;
    snprintf(p, sizeof(p), "%s/quant_rows.json", argv[1]);
    if (!rows_fixture(p, grid)) return 1;
    g_state = 0x5eed0002ull;
    snprintf(p, sizeof(p), "%s/router_select.json", argv[1]);
    if (!router_fixture(p)) return 1;
    g_state = 0x5eed0003ull;
    snprintf(p, sizeof(p), "%s/shared_expert.json", argv[1]);
    snprintf(t, sizeof(t), "%s/.shared_tmp.bin", argv[1]);
    if (!shared_fixture(p, t)) return 1;
    snprintf(p, sizeof(p), "%s/f16.json", argv[1]);
    if (!f16_fixture(p)) return 1;
    printf("golden fixtures written to %s\n", argv[1]);
    return 0;
}
