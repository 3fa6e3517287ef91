/*
 * TEST INFRASTRUCTURE - golden vectors for the IQ2_XS (17) and IQ1_M (29) routed-expert formats.
 *
 * Links against oracle/_ref/libref.so (the reference's own C, compiled where it lies) and writes
 *   iq_grids.json      the two codebooks the reference hands to its kernels (rl_native_quant_tables_init,
 *                      native/redlite_native_tables.c), as int8 hex, with the reference's own FNV-1a of each
 *   quant_rows_xs_m.json   rl_native_quant_row_dot (native/redlite_native_reference.c:182-195) on seeded rows
 * Floats and doubles are little-endian hex.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "redlite_native_reference.h"
#include "redlite_native_tables.h"

static uint64_t g_state;
static uint32_t rnd32(void) {
    uint64_t z = (g_state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return (uint32_t)((z ^ (z >> 31)) >> 32);
}
static float rnd_unit(void) { return (float)(rnd32() >> 8) * (1.0f / 16777216.0f); }
static float rnd_normal(void) {
    float s = 0.0f;
    for (int i = 0; i < 12; ++i) s += rnd_unit();
    return s - 6.0f;
}
static void hex(FILE *f, const char *key, const void *data, size_t n, int last) {
    const uint8_t *p = (const uint8_t *)data;
    fprintf(f, "\"%s\": \"", key);
    for (size_t i = 0; i < n; ++i) fprintf(f, "%02x", p[i]);
    fprintf(f, "\"%s", last ? "" : ", ");
}
static uint16_t half_bits_from_float(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    const int32_t e = (int32_t)((b >> 23) & 255u) - 127 + 15;
    if (e <= 0) return 0;
    return (uint16_t)(((b >> 16) & 0x8000u) | ((uint32_t)e << 10) | ((b & 0x7fffffu) >> 13));
}

enum { FILL_RANDOM = 0, FILL_ZERO, FILL_ONES, FILL_SUBNORMAL_D, FILL_NEG_D };

/* every bit pattern is a valid block; only the fp16 d is steered: IQ2_XS keeps it in bytes 0..1, IQ1_M spreads it over
 * the top nibbles of its four 16-bit scale words (bytes 48..55) */
static void fill_row(uint32_t type, uint32_t ncols, int mode, uint8_t *row) {
    const size_t bb = type == 17u ? 74u : 56u;
    for (uint32_t b = 0; b < ncols / 256u; ++b) {
        uint8_t *bp = row + b * bb;
        for (size_t i = 0; i < bb; ++i) bp[i] = mode == FILL_ZERO ? 0u : mode == FILL_ONES ? 0xffu : (uint8_t)rnd32();
        uint16_t d = half_bits_from_float(1e-3f + rnd_unit() * (2e-2f - 1e-3f));
        if (mode == FILL_SUBNORMAL_D) d = (uint16_t)(1u + (rnd32() % 1023u));
        if (mode == FILL_NEG_D) d |= 0x8000u;
        if (mode == FILL_ZERO || mode == FILL_ONES) d = 0x3c00u;
        if (type == 17u) {
            bp[0] = (uint8_t)(d & 255u);
            bp[1] = (uint8_t)(d >> 8);
        } else {
            for (uint32_t i = 0; i < 4u; ++i) {
                uint16_t sc = (uint16_t)(bp[48u + 2u * i] | (bp[49u + 2u * i] << 8));
                sc = (uint16_t)((sc & 0x0fffu) | (((d >> (4u * i)) & 15u) << 12));
                bp[48u + 2u * i] = (uint8_t)(sc & 255u);
                bp[49u + 2u * i] = (uint8_t)(sc >> 8);
            }
        }
    }
}

int main(int argc, char **argv) {
    if (argc != 2) { fprintf(stderr, "usage: %s <output dir>\n", argv[0]); return 2; }
    rl_native_quant_tables tab;
    char err[256] = {0}, p[512];
    if (!rl_native_quant_tables_init(&tab, err, sizeof(err))) { fprintf(stderr, "tables: %s\n", err); return 1; }
    snprintf(p, sizeof(p), "%s/iq_grids.json", argv[1]);
    FILE *f = fopen(p, "w");
    if (!f) { perror(p); return 1; }
    fprintf(f, "{\"about\": \"codebooks of rl_native_quant_tables_init: 512 x 8 (IQ2_XS) and 2048 x 8 (IQ1_M) int8 values, hex; fnv1a as the reference computes it\",\n ");
    fprintf(f, "\"iq2_xs_fnv1a\": \"%016llx\", \"iq1_m_fnv1a\": \"%016llx\",\n ",
            (unsigned long long)rl_native_quant_table_fnv1a(tab.iq2_xs, RL_IQ2_XS_GRID_COUNT),
            (unsigned long long)rl_native_quant_table_fnv1a(tab.iq1_m, RL_IQ1_M_GRID_COUNT));
    hex(f, "iq2_xs", tab.iq2_xs, RL_IQ2_XS_GRID_COUNT, 0);
    fprintf(f, "\n ");
    hex(f, "iq1_m", tab.iq1_m, RL_IQ1_M_GRID_COUNT, 1);
    fprintf(f, "}\n");
    fclose(f);

    g_state = 0x5eed0017ull;
    snprintf(p, sizeof(p), "%s/quant_rows_xs_m.json", argv[1]);
    f = fopen(p, "w");
    if (!f) { perror(p); return 1; }
    fprintf(f, "{\"about\": \"reference rl_native_quant_row_dot on seeded IQ2_XS (17) / IQ1_M (29) rows\",\n \"cases\": [\n");
    const uint32_t types[2] = {17u, 29u}, widths[3] = {256u, 512u, 2048u};
    const int modes[5] = {FILL_RANDOM, FILL_ZERO, FILL_ONES, FILL_SUBNORMAL_D, FILL_NEG_D};
    int first = 1;
    for (int ti = 0; ti < 2; ++ti) for (int wi = 0; wi < 3; ++wi) for (int mi = 0; mi < 5; ++mi) {
        if (mi > 0 && wi != 1) continue;
        const int reps = mi == 0 ? 3 : 1;
        for (int rep = 0; rep < reps; ++rep) {
            const uint32_t type = types[ti], ncols = widths[wi];
            const size_t rb = rl_native_row_bytes(type, ncols);
            uint8_t *row = (uint8_t *)malloc(rb);
            float *x = (float *)malloc(sizeof(float) * ncols);
            fill_row(type, ncols, modes[mi], row);
            for (uint32_t i = 0; i < ncols; ++i) x[i] = rnd_normal();
            double dot = 0.0;
            const int8_t *grid = type == 17u ? tab.iq2_xs : tab.iq1_m;
            const size_t gc = type == 17u ? RL_IQ2_XS_GRID_COUNT : RL_IQ1_M_GRID_COUNT;
            if (!rl_native_quant_row_dot(row, rb, type, x, ncols, grid, gc, &dot, err, sizeof(err))) { fprintf(stderr, "row dot: %s\n", err); return 1; }
            fprintf(f, "%s  {\"type\": %u, \"ncols\": %u, \"fill\": %d, ", first ? "" : ",\n", type, ncols, modes[mi]);
            hex(f, "row", row, rb, 0);
            hex(f, "x", x, sizeof(float) * ncols, 0);
            hex(f, "dot", &dot, 8, 1);
            fprintf(f, "}");
            first = 0;
            free(row); free(x);
        }
    }
    fprintf(f, "\n ]}\n");
    fclose(f);
    rl_native_quant_tables_free(&tab);
    printf("IQ2_XS / IQ1_M fixtures written to %s\n", argv[1]);
    return 0;
}
