/*
 * TEST INFRASTRUCTURE - CPU oracle for the routed-expert MoE FFN path.
 * See moe_oracle.h for what this is and is not. Reference paths are relative
 * to the reference repository root.
 */
#define _POSIX_C_SOURCE 200809L
#include "moe_oracle.h"
#include "moe_oracle_tables.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define QK 256u
#define BLK_Q6K 210u
#define BLK_IQ2XXS 66u
#define BLK_IQ3S 110u

static uint16_t le16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static uint32_t le32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* native/redlite_native_quant_cpu.c:20-38 - exact IEEE binary16 -> binary32, subnormals normalised by shifting */
float orc_f16_to_f32(uint16_t h) {
    const uint32_t s = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 1023u;
    uint32_t u;
    if (e == 31u) u = s | 0x7f800000u | (m << 13);
    else if (e != 0u) u = s | ((e + 112u) << 23) | (m << 13);
    else if (m == 0u) u = s;
    else {
        uint32_t ex = 113u;               /* exponent of 2^-14 */
        while (!(m & 1024u)) { m <<= 1; --ex; }
        u = s | (ex << 23) | ((m & 1023u) << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void orc_f16_all(float *out) { for (uint32_t h = 0; h < 65536u; ++h) out[h] = orc_f16_to_f32((uint16_t)h); }

const uint8_t *orc_iq2xxs_grid(void) { return orc_iq2xxs_grid_bytes; }
const uint32_t *orc_iq3s_grid(void) { return orc_iq3s_grid_words; }

uint32_t orc_crc32(const void *data, size_t n) {
    const uint8_t *p = (const uint8_t *)data;
    uint32_t c = 0xffffffffu;
    for (size_t i = 0; i < n; ++i) {
        c ^= p[i];
        for (int k = 0; k < 8; ++k) c = (c >> 1) ^ (0xedb88320u & (0u - (c & 1u)));
    }
    return c ^ 0xffffffffu;
}

/* native/redlite_native_shared_exec.c:70-76, native/redlite_native_iq3.c:35-52 */
size_t orc_block_bytes(uint32_t type) {
    switch (type) {
        case ORC_TYPE_Q6_K: return BLK_Q6K;
        case ORC_TYPE_IQ2_XXS: return BLK_IQ2XXS;
        case ORC_TYPE_IQ3_S: return BLK_IQ3S;
        case 17u: return 74u;       /* IQ2_XS, native/redlite_native_reference.c:116 */
        case 29u: return 56u;       /* IQ1_M, native/redlite_native_reference.c:144 */
        default: return 0;
    }
}

size_t orc_row_bytes(uint32_t type, uint32_t ncols) {
    if (!ncols) return 0;
    if (type == ORC_TYPE_F32) return (size_t)ncols * 4u;
    const size_t b = orc_block_bytes(type);
    if (!b || ncols % QK) return 0;
    return (size_t)(ncols / QK) * b;
}

/* sign byte of an IQ2_XXS entry: the seven stored bits plus their parity as bit 7
 * (native/redlite_native_quant_cpu.c:182-183, native/redlite_native_shared_exec.c:59-68,134) */
static uint32_t sign8_from7(uint32_t s7) { return s7 | (((uint32_t)__builtin_popcount(s7 & 127u) & 1u) << 7); }

/* ---- dequantisation to f32, value for value ---- */

/* native/redlite_native_quant_cpu.c:166-191 */
static void deq_iq2xxs_block(const uint8_t *bp, float *y) {
    const float d = orc_f16_to_f32(le16(bp));
    for (uint32_t g = 0; g < 8u; ++g) {
        const uint32_t idx4 = le32(bp + 2u + 8u * g);
        const uint32_t aux = le32(bp + 6u + 8u * g);
        const float db = d * (0.5f + (float)(aux >> 28)) * 0.25f;
        for (uint32_t l = 0; l < 4u; ++l) {
            const uint8_t *mag = orc_iq2xxs_grid_bytes + 8u * ((idx4 >> (8u * l)) & 255u);
            const uint32_t sg = sign8_from7((aux >> (7u * l)) & 127u);
            for (uint32_t j = 0; j < 8u; ++j)
                y[32u * g + 8u * l + j] = db * (float)mag[j] * (((sg >> j) & 1u) ? -1.0f : 1.0f);
        }
    }
}

/* native/redlite_native_iq3.c:82-91 (one group of 8), :112-118 (row) */
static void deq_iq3s_group(const uint8_t *bp, uint32_t g, float out[8]) {
    const float d = orc_f16_to_f32(le16(bp));
    const uint32_t sub = g >> 2, l = g & 3u;
    const uint8_t *qs = bp + 2u + 8u * sub;
    const uint32_t qh = bp[66u + sub];
    const uint32_t sg = bp[74u + 4u * sub + l];
    const uint32_t nib = (bp[106u + (sub >> 1)] >> (4u * (sub & 1u))) & 15u;
    const float db = d * (float)(1 + 2 * (int)nib);
    const uint32_t ia = qs[2u * l] | ((qh << (8u - 2u * l)) & 256u);
    const uint32_t ib = qs[2u * l + 1u] | ((qh << (7u - 2u * l)) & 256u);
    const uint32_t wa = orc_iq3s_grid_words[ia], wb = orc_iq3s_grid_words[ib];
    for (uint32_t j = 0; j < 4u; ++j) {
        out[j] = db * (float)((wa >> (8u * j)) & 255u) * (((sg >> j) & 1u) ? -1.f : 1.f);
        out[4u + j] = db * (float)((wb >> (8u * j)) & 255u) * (((sg >> (4u + j)) & 1u) ? -1.f : 1.f);
    }
}

/* native/redlite_native_quant_cpu.c:130-153 */
static void deq_q6k_block(const uint8_t *bp, float *y) {
    const float d = orc_f16_to_f32(le16(bp + 208u));
    for (uint32_t half = 0; half < 2u; ++half) {
        const uint8_t *ql = bp + 64u * half;
        const uint8_t *qh = bp + 128u + 32u * half;
        const int8_t *sc = (const int8_t *)(bp + 192u + 8u * half);
        float *o = y + 128u * half;
        for (uint32_t l = 0; l < 32u; ++l) {
            const uint32_t is = l >> 4;
            const int8_t q1 = (int8_t)((ql[l] & 15u) | (((qh[l] >> 0) & 3u) << 4)) - 32;
            const int8_t q2 = (int8_t)((ql[l + 32u] & 15u) | (((qh[l] >> 2) & 3u) << 4)) - 32;
            const int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3u) << 4)) - 32;
            const int8_t q4 = (int8_t)((ql[l + 32u] >> 4) | (((qh[l] >> 6) & 3u) << 4)) - 32;
            o[l] = d * (float)sc[is] * (float)q1;
            o[l + 32u] = d * (float)sc[is + 2u] * (float)q2;
            o[l + 64u] = d * (float)sc[is + 4u] * (float)q3;
            o[l + 96u] = d * (float)sc[is + 6u] * (float)q4;
        }
    }
}

/* ---- IQ2_XS / IQ1_M, native/redlite_native_reference.c:60-172 ---- */

static uint32_t rd16(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

/* weight i (0..255) of one block as the double the reference multiplies the activation with */
static double xs_m_weight(uint32_t type, const uint8_t *bp, const int8_t *grid, uint32_t i) {
    if (type == 17u) {                                             /* :122-142 */
        const double d = (double)orc_f16_to_f32((uint16_t)rd16(bp));
        const uint32_t group = i >> 4, part = (i >> 3) & 1u, j = i & 7u;
        const uint32_t scale = (bp[66u + (group >> 1)] >> (4u * (group & 1u))) & 0x0fu;
        const double db = d * (0.5 + (double)scale) * 0.25;
        const uint32_t q = rd16(bp + 2u + 2u * (2u * group + part));
        uint32_t s7 = (q >> 9) & 0x7fu, parity = 0u;
        for (uint32_t v = s7; v; v >>= 1) parity ^= v & 1u;       /* sign_byte, :60-69 */
        const uint32_t signs = s7 | (parity << 7);
        return db * (double)grid[(q & 0x01ffu) * 8u + j] * ((signs >> j) & 1u ? -1.0 : 1.0);
    }
    /* IQ1_M, :149-170 */
    uint32_t sc[4];
    for (uint32_t k = 0; k < 4u; ++k) sc[k] = rd16(bp + 48u + 2u * k);
    const uint32_t d_bits = (sc[0] >> 12) | ((sc[1] >> 8) & 0x00f0u) | ((sc[2] >> 4) & 0x0f00u) | (sc[3] & 0xf000u);
    const double d = (double)orc_f16_to_f32((uint16_t)d_bits);
    const uint32_t group = i >> 3, j = i & 7u;
    const uint32_t nibble = (bp[32u + (group >> 1)] >> (4u * (group & 1u))) & 0x0fu;
    const uint32_t grid_index = (uint32_t)bp[group] | ((nibble & 7u) << 8);
    const double delta = (nibble & 8u) ? -0.125 : 0.125;
    const uint32_t scale_index = group >> 1, scale = (sc[scale_index >> 2] >> (3u * (scale_index & 3u))) & 7u;
    return d * (double)(2u * scale + 1u) * ((double)grid[grid_index * 8u + j] + delta);
}

int orc_dequant_row_grid(uint32_t type, const uint8_t *row, uint32_t ncols, const int8_t *grid, float *out) {
    if (!row || !grid || !out || !ncols || ncols % QK || (type != 17u && type != 29u)) return 0;
    const size_t bb = type == 17u ? 74u : 56u;
    for (uint32_t i = 0; i < ncols; ++i) out[i] = (float)xs_m_weight(type, row + (size_t)(i / QK) * bb, grid, i % QK);
    return 1;
}

/* The caller's codebooks kept for the functions that take no grid argument (row dots, matvec, expert and layer forward), the way
 * the reference keeps rl_native_quant_tables beside its model (native/redlite_native_reference.c:343). */
static int8_t g_xs_grid[512 * 8], g_m_grid[2048 * 8];
static int g_have_xs = 0, g_have_m = 0;

void orc_set_codebooks(const int8_t *iq2_xs, const int8_t *iq1_m) {
    if (iq2_xs) { memcpy(g_xs_grid, iq2_xs, sizeof(g_xs_grid)); g_have_xs = 1; }
    if (iq1_m) { memcpy(g_m_grid, iq1_m, sizeof(g_m_grid)); g_have_m = 1; }
}

static const int8_t *kept_grid(uint32_t type) {
    return type == 17u ? (g_have_xs ? g_xs_grid : NULL) : type == 29u ? (g_have_m ? g_m_grid : NULL) : NULL;
}

int orc_row_dot_grid(uint32_t type, const uint8_t *row, const float *x, uint32_t ncols, const int8_t *grid, double *out) {
    if (!row || !grid || !x || !out || !ncols || ncols % QK || (type != 17u && type != 29u)) return 0;
    const size_t bb = type == 17u ? 74u : 56u;
    double acc = 0.0;
    for (uint32_t i = 0; i < ncols; ++i) acc += (double)x[i] * xs_m_weight(type, row + (size_t)(i / QK) * bb, grid, i % QK);
    *out = acc;
    return 1;
}

/* native/redlite_native_quant_cpu.c:155-196 (types 0, 14, 16 and the IQ3 delegation) */
int orc_dequant_row(uint32_t type, const uint8_t *row, uint32_t ncols, float *out) {
    if (!row || !out || !ncols) return 0;
    if (type == ORC_TYPE_F32) { memcpy(out, row, (size_t)ncols * 4u); return 1; }
    if (ncols % QK || !orc_block_bytes(type)) return 0;
    if (type == 17u || type == 29u) return orc_dequant_row_grid(type, row, ncols, kept_grid(type), out);
    for (uint32_t b = 0; b < ncols / QK; ++b) {
        float *y = out + (size_t)b * QK;
        if (type == ORC_TYPE_IQ2_XXS) deq_iq2xxs_block(row + (size_t)b * BLK_IQ2XXS, y);
        else if (type == ORC_TYPE_Q6_K) deq_q6k_block(row + (size_t)b * BLK_Q6K, y);
        else for (uint32_t g = 0; g < 32u; ++g) deq_iq3s_group(row + (size_t)b * BLK_IQ3S, g, y + 8u * g);
    }
    return 1;
}

/* ---- row dot products, double accumulation, one weight at a time in column order ---- */

/* native/redlite_native_shared_exec.c:111-145 - the weight is formed in double */
static double dot_iq2xxs(const uint8_t *row, const float *xf, const double *xd, uint32_t ncols) {
    double acc = 0.0;
    for (uint32_t b = 0; b < ncols / QK; ++b) {
        const uint8_t *bp = row + (size_t)b * BLK_IQ2XXS;
        const float d = orc_f16_to_f32(le16(bp));
        for (uint32_t g = 0; g < 8u; ++g) {
            const uint32_t idx4 = le32(bp + 2u + 8u * g);
            const uint32_t aux = le32(bp + 6u + 8u * g);
            const double db = (double)d * (0.5 + (double)(aux >> 28)) * 0.25;
            for (uint32_t l = 0; l < 4u; ++l) {
                const uint8_t *mag = orc_iq2xxs_grid_bytes + 8u * ((idx4 >> (8u * l)) & 255u);
                const uint32_t sg = sign8_from7((aux >> (7u * l)) & 127u);
                const uint32_t c = b * QK + 32u * g + 8u * l;
                for (uint32_t j = 0; j < 8u; ++j) {
                    const double w = db * (double)mag[j] * (((sg >> j) & 1u) ? -1.0 : 1.0);
                    acc += (xd ? xd[c + j] : (double)xf[c + j]) * w;
                }
            }
        }
    }
    return acc;
}

/* native/redlite_native_shared_exec.c:78-109 - four interleaved quants per l, weight formed in double */
static double dot_q6k(const uint8_t *row, const float *xf, const double *xd, uint32_t ncols) {
    double acc = 0.0;
    for (uint32_t b = 0; b < ncols / QK; ++b) {
        const uint8_t *bp = row + (size_t)b * BLK_Q6K;
        const float d = orc_f16_to_f32(le16(bp + 208u));
        for (uint32_t half = 0; half < 2u; ++half) {
            const uint8_t *ql = bp + 64u * half;
            const uint8_t *qh = bp + 128u + 32u * half;
            const int8_t *sc = (const int8_t *)(bp + 192u + 8u * half);
            const uint32_t c = b * QK + 128u * half;
            for (uint32_t l = 0; l < 32u; ++l) {
                const uint32_t is = l >> 4;
                const int q1 = (int)((ql[l] & 15u) | (((qh[l] >> 0) & 3u) << 4)) - 32;
                const int q2 = (int)((ql[l + 32u] & 15u) | (((qh[l] >> 2) & 3u) << 4)) - 32;
                const int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3u) << 4)) - 32;
                const int q4 = (int)((ql[l + 32u] >> 4) | (((qh[l] >> 6) & 3u) << 4)) - 32;
#define X(i) (xd ? xd[(i)] : (double)xf[(i)])
                acc += X(c + l) * ((double)d * sc[is] * q1);
                acc += X(c + l + 32u) * ((double)d * sc[is + 2u] * q2);
                acc += X(c + l + 64u) * ((double)d * sc[is + 4u] * q3);
                acc += X(c + l + 96u) * ((double)d * sc[is + 6u] * q4);
#undef X
            }
        }
    }
    return acc;
}

/* native/redlite_native_iq3.c:120-148 - the f32 dequantised value times the input, summed in double */
static double dot_iq3s(const uint8_t *row, const float *xf, const double *xd, uint32_t ncols) {
    double acc = 0.0;
    float v[8];
    for (uint32_t b = 0; b < ncols / QK; ++b)
        for (uint32_t g = 0; g < 32u; ++g) {
            deq_iq3s_group(row + (size_t)b * BLK_IQ3S, g, v);
            const uint32_t c = b * QK + 8u * g;
            for (uint32_t j = 0; j < 8u; ++j) acc += (double)v[j] * (xd ? xd[c + j] : (double)xf[c + j]);
        }
    return acc;
}

static int dot_any(uint32_t type, const uint8_t *row, const float *xf, const double *xd, uint32_t ncols, double *out) {
    if (!row || (!xf && !xd) || !out || !ncols) return 0;
    if (type == ORC_TYPE_F32) {     /* native/redlite_native_quant_cpu.c:203, native/redlite_native_engine_cpu.c:349-353 */
        double acc = 0.0;
        for (uint32_t i = 0; i < ncols; ++i) {
            float w;
            memcpy(&w, row + 4u * (size_t)i, 4);
            acc += (double)w * (xd ? xd[i] : (double)xf[i]);
        }
        *out = acc;
        return 1;
    }
    if (ncols % QK) return 0;
    if (type == ORC_TYPE_IQ2_XXS) *out = dot_iq2xxs(row, xf, xd, ncols);
    else if (type == ORC_TYPE_Q6_K) *out = dot_q6k(row, xf, xd, ncols);
    else if (type == ORC_TYPE_IQ3_S) *out = dot_iq3s(row, xf, xd, ncols);
    else if (type == 17u || type == 29u) {       /* native/redlite_native_reference.c:78-172 */
        const int8_t *grid = kept_grid(type);
        if (!grid) return 0;
        const size_t bb = orc_block_bytes(type);
        double acc = 0.0;
        for (uint32_t i = 0; i < ncols; ++i)
            acc += (xd ? xd[i] : (double)xf[i]) * xs_m_weight(type, row + (size_t)(i / QK) * bb, grid, i % QK);
        *out = acc;
    } else return 0;
    return 1;
}

/* native/redlite_native_quant_cpu.c:198-280 */
int orc_row_dot(uint32_t type, const uint8_t *row, const float *x, uint32_t ncols, double *out) {
    return dot_any(type, row, x, NULL, ncols, out);
}

/* native/redlite_native_iq3.c:135-148 for IQ3_S. For IQ2_XXS / Q6_K the reference has no double-input
 * variant; the same per-weight formulas are used with the input taken as double. */
int orc_row_dot_d(uint32_t type, const uint8_t *row, const double *x, uint32_t ncols, double *out) {
    return dot_any(type, row, NULL, x, ncols, out);
}

/* ---- rows over pthreads: contiguous chunks, threads created and joined per call
 *      (native/redlite_native_engine_cpu.c:42-92) ---- */

typedef struct {
    uint32_t type, ncols, begin, end;
    const uint8_t *w;
    size_t rb;
    const float *xf;
    const double *xd;
    float *of;
    double *od;
    int ok;
} rows_job;

static void *rows_run(void *p) {
    rows_job *j = (rows_job *)p;
    j->ok = 1;
    for (uint32_t r = j->begin; r < j->end; ++r) {
        double v = 0.0;
        if (!dot_any(j->type, j->w + (size_t)r * j->rb, j->xf, j->xd, j->ncols, &v)) { j->ok = 0; break; }
        if (j->of) j->of[r] = (float)v;
        if (j->od) j->od[r] = v;
    }
    return NULL;
}

/* rows [0,count) of the matrix starting at w (already offset to row_start); results indexed from 0 */
static int rows_mt(uint32_t type, const uint8_t *w, uint32_t ncols, uint32_t count,
                   const float *xf, const double *xd, float *of, double *od, int threads) {
    const size_t rb = orc_row_bytes(type, ncols);
    if (!rb || !w || !count) return 0;
    if (threads > 64) threads = 64;
    if ((uint32_t)threads > count) threads = (int)count;
    if (threads < 1) threads = 1;
    rows_job jobs[64];
    pthread_t tid[64];
    int live[64] = {0};
    const uint32_t chunk = (count + (uint32_t)threads - 1u) / (uint32_t)threads;
    for (int i = 0; i < threads; ++i) {
        rows_job *j = &jobs[i];
        j->type = type; j->ncols = ncols; j->w = w; j->rb = rb; j->xf = xf; j->xd = xd; j->of = of; j->od = od; j->ok = 1;
        j->begin = (uint32_t)i * chunk;
        j->end = j->begin + chunk > count ? count : j->begin + chunk;
        if (j->begin > count) j->begin = count;
        if (i > 0) live[i] = pthread_create(&tid[i], NULL, rows_run, j) == 0;
    }
    rows_run(&jobs[0]);
    int ok = jobs[0].ok;
    for (int i = 1; i < threads; ++i) {
        if (live[i]) pthread_join(tid[i], NULL); else rows_run(&jobs[i]);
        ok = ok && jobs[i].ok;
    }
    return ok;
}

int orc_matvec(uint32_t type, const uint8_t *w, uint32_t ncols, uint32_t row_start, uint32_t row_count,
               const float *x, float *out, int threads) {
    const size_t rb = orc_row_bytes(type, ncols);
    if (!rb || !w || !x || !out) return 0;
    return rows_mt(type, w + (size_t)row_start * rb, ncols, row_count, x, NULL, out, NULL, threads);
}

/* native/redlite_native_engine_cpu.c:96-101 */
void orc_rmsnorm(const float *x, const float *w, uint32_t n, float eps, float *out) {
    double ss = 0.0;
    for (uint32_t i = 0; i < n; ++i) ss += (double)x[i] * x[i];
    const double inv = 1.0 / sqrt(ss / n + (double)eps);
    for (uint32_t i = 0; i < n; ++i) out[i] = (float)((double)x[i] * inv * (w ? w[i] : 1.0f));
}

/* ---- router ---- */

/* native/redlite_native_engine_cpu.c:347-355 (F32). A quantised router row goes through the dense row dot
 * (native/redlite_native_quant_cpu.c:198-280), result rounded to float like every matvec output (:62). */
int orc_router_logits(uint32_t type, const uint8_t *w, uint32_t hidden, uint32_t experts, const float *x, float *logits) {
    if (!w || !x || !logits || !experts) return 0;
    return rows_mt(type, w, hidden, experts, x, NULL, logits, NULL, 1);
}

/* native/redlite_native_router_exec.c:102-184 */
int orc_router_select(const float *logits, uint32_t experts, uint32_t top_k, uint32_t *ids, float *weights, float *probs) {
    if (!logits || !ids || !weights || !experts || !top_k || top_k > experts) return 0;
    float *p = probs ? probs : (float *)malloc((size_t)experts * sizeof(float));
    unsigned char *taken = (unsigned char *)calloc(experts, 1);
    int ok = 0;
    if (!p || !taken) goto out;
    float mx = logits[0];
    for (uint32_t i = 1; i < experts; ++i) if (logits[i] > mx) mx = logits[i];
    double den = 0.0;
    for (uint32_t i = 0; i < experts; ++i) { p[i] = expf(logits[i] - mx); den += (double)p[i]; }
    if (!(den > 0.0) || !isfinite(den)) goto out;
    const float inv = (float)(1.0 / den);
    for (uint32_t i = 0; i < experts; ++i) p[i] *= inv;
    double picked = 0.0;
    for (uint32_t k = 0; k < top_k; ++k) {
        uint32_t arg = UINT32_MAX;
        float best = -INFINITY;
        for (uint32_t i = 0; i < experts; ++i) {
            if (taken[i]) continue;
            if (arg == UINT32_MAX || p[i] > best || (p[i] == best && i < arg)) { arg = i; best = p[i]; }
        }
        if (arg == UINT32_MAX) goto out;
        taken[arg] = 1;
        ids[k] = arg;
        weights[k] = best;
        picked += (double)best;
    }
    if (!(picked > 0.0) || !isfinite(picked)) goto out;
    const float invp = (float)(1.0 / picked);
    for (uint32_t k = 0; k < top_k; ++k) weights[k] *= invp;
    ok = 1;
out:
    free(taken);
    if (!probs) free(p);
    return ok;
}

/* ---- experts ---- */

/* native/redlite_native_reference.c:251-259 */
double orc_silu_mul(double gate, double up) {
    double s;
    if (gate >= 0.0) s = 1.0 / (1.0 + exp(-gate));
    else { const double e = exp(gate); s = e / (1.0 + e); }
    return (gate * s) * up;
}

static int expert_ffn_mt(uint32_t gu_type, uint32_t dn_type, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                         uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count,
                         const float *x, double *out, int threads) {
    const size_t drb = orc_row_bytes(dn_type, ffn);
    if (!gate || !up || !down || !x || !out || !drb || !row_count || row_start >= hidden || row_count > hidden - row_start) return 0;
    double *g = (double *)malloc(sizeof(double) * 3u * (size_t)ffn);
    if (!g) return 0;
    double *u = g + ffn, *a = u + ffn;
    int ok = rows_mt(gu_type, gate, hidden, ffn, x, NULL, NULL, g, threads) &&
             rows_mt(gu_type, up, hidden, ffn, x, NULL, NULL, u, threads);
    if (ok) {
        for (uint32_t i = 0; i < ffn; ++i) a[i] = orc_silu_mul(g[i], u[i]);
        ok = rows_mt(dn_type, down + (size_t)row_start * drb, ffn, row_count, NULL, a, NULL, out, threads);
    }
    free(g);
    return ok;
}

/* native/redlite_native_reference.c:267-305 */
int orc_expert_ffn(uint32_t gate_up_type, uint32_t down_type, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                   uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count, const float *x, double *out) {
    return expert_ffn_mt(gate_up_type, down_type, gate, up, down, hidden, ffn, row_start, row_count, x, out, 1);
}

static int routed_topk_mt(uint32_t gu_type, uint32_t dn_type,
                          const uint8_t *gate_base, const uint8_t *up_base, const uint8_t *down_base,
                          size_t gate_stride, size_t up_stride, size_t down_stride,
                          const uint32_t *ids, const float *weights, uint32_t top_k,
                          uint32_t hidden, uint32_t ffn, const float *x, double *out, int threads) {
    if (!ids || !weights || !top_k || !out) return 0;
    double *tmp = (double *)malloc(sizeof(double) * (size_t)hidden);
    if (!tmp) return 0;
    for (uint32_t r = 0; r < hidden; ++r) out[r] = 0.0;
    int ok = 1;
    for (uint32_t k = 0; k < top_k && ok; ++k) {
        const size_t e = ids[k];
        ok = expert_ffn_mt(gu_type, dn_type, gate_base + e * gate_stride, up_base + e * up_stride, down_base + e * down_stride,
                           hidden, ffn, 0u, hidden, x, tmp, threads);
        if (ok) for (uint32_t r = 0; r < hidden; ++r) out[r] += (double)weights[k] * tmp[r];
    }
    free(tmp);
    return ok;
}

/* one row dot for any pool type: the two codebook formats go through the caller's grids (native/redlite_native_reference.c:78-172,
 * float or double activations), the rest through dot_any */
static int pool_row_dot(uint32_t type, const uint8_t *row, const float *xf, const double *xd, uint32_t ncols,
                        const int8_t *xs_grid, const int8_t *m_grid, double *out) {
    if (type != 17u && type != 29u) return dot_any(type, row, xf, xd, ncols, out);
    const int8_t *grid = type == 17u ? xs_grid : m_grid;
    if (!grid || ncols % QK) return 0;
    const size_t bb = type == 17u ? 74u : 56u;
    double acc = 0.0;
    for (uint32_t i = 0; i < ncols; ++i)
        acc += (xd ? xd[i] : (double)xf[i]) * xs_m_weight(type, row + (size_t)(i / QK) * bb, grid, i % QK);
    *out = acc;
    return 1;
}

static size_t pool_row_bytes(uint32_t type, uint32_t ncols) {
    if (type == 17u || type == 29u) return ncols % QK ? 0u : (size_t)(ncols / QK) * (type == 17u ? 74u : 56u);
    return orc_row_bytes(type, ncols);
}

/* native/redlite_native_reference.c:267-305 with the codebook formats (types 17 and 29) allowed on either side */
int orc_expert_ffn_grid(uint32_t gate_up_type, uint32_t down_type, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                        uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count, const float *x,
                        const int8_t *xs_grid, const int8_t *m_grid, double *out) {
    const size_t grb = pool_row_bytes(gate_up_type, hidden), drb = pool_row_bytes(down_type, ffn);
    if (!gate || !up || !down || !x || !out || !grb || !drb || !row_count || row_start >= hidden || row_count > hidden - row_start) return 0;
    double *a = (double *)malloc(sizeof(double) * (size_t)ffn);
    if (!a) return 0;
    int ok = 1;
    for (uint32_t i = 0; i < ffn && ok; ++i) {
        double g = 0.0, u = 0.0;
        ok = pool_row_dot(gate_up_type, gate + (size_t)i * grb, x, NULL, hidden, xs_grid, m_grid, &g) &&
             pool_row_dot(gate_up_type, up + (size_t)i * grb, x, NULL, hidden, xs_grid, m_grid, &u);
        a[i] = orc_silu_mul(g, u);
    }
    for (uint32_t r = 0; r < row_count && ok; ++r)
        ok = pool_row_dot(down_type, down + (size_t)(row_start + r) * drb, NULL, a, ffn, xs_grid, m_grid, &out[r]);
    free(a);
    return ok;
}

/* native/redlite_native_reference.c:344-372 */
int orc_routed_topk(uint32_t gate_up_type, uint32_t down_type,
                    const uint8_t *gate_base, const uint8_t *up_base, const uint8_t *down_base,
                    size_t gate_stride, size_t up_stride, size_t down_stride,
                    const uint32_t *ids, const float *weights, uint32_t top_k,
                    uint32_t hidden, uint32_t ffn, const float *x, double *out) {
    return routed_topk_mt(gate_up_type, down_type, gate_base, up_base, down_base, gate_stride, up_stride, down_stride,
                          ids, weights, top_k, hidden, ffn, x, out, 1);
}

/* native/redlite_native_engine_cpu.c:367-378 */
int orc_shared_expert(uint32_t gate_up_type, uint32_t down_type,
                      const uint8_t *gate, const uint8_t *up, const uint8_t *down, const float *gate_inp,
                      uint32_t hidden, uint32_t ffn, const float *x, float *out_sh, double *scalar, int threads) {
    if (!gate || !up || !down || !gate_inp || !x || !out_sh || !scalar) return 0;
    float *g = (float *)malloc(sizeof(float) * 3u * (size_t)ffn);
    if (!g) return 0;
    float *u = g + ffn, *a = u + ffn;
    int ok = rows_mt(gate_up_type, gate, hidden, ffn, x, NULL, g, NULL, threads) &&
             rows_mt(gate_up_type, up, hidden, ffn, x, NULL, u, NULL, threads);
    if (ok) {
        for (uint32_t i = 0; i < ffn; ++i) {
            const double gv = g[i];
            a[i] = (float)((gv / (1.0 + exp(-gv))) * (double)u[i]);
        }
        ok = rows_mt(down_type, down, ffn, hidden, a, NULL, out_sh, NULL, threads);
    }
    if (ok) {
        double acc = 0.0;
        for (uint32_t i = 0; i < hidden; ++i) acc += (double)gate_inp[i] * x[i];
        *scalar = 1.0 / (1.0 + exp(-acc));
    }
    free(g);
    return ok;
}

static double sigmoid_stable(double v) {
    if (v >= 0.0) return 1.0 / (1.0 + exp(-v));
    const double z = exp(v);
    return z / (1.0 + z);
}

/* native/redlite_native_shared_exec.c:228-314 */
int orc_shared_expert_standalone(uint32_t gate_up_type, uint32_t down_type,
                      const uint8_t *gate, const uint8_t *up, const uint8_t *down, const float *gate_inp,
                      uint32_t hidden, uint32_t ffn, uint32_t row_start, uint32_t row_count,
                      const float *x, double *out, double *scalar) {
    const size_t grb = orc_row_bytes(gate_up_type, hidden), drb = orc_row_bytes(down_type, ffn);
    if (!gate || !up || !down || !gate_inp || !x || !out || !grb || !drb || !row_count ||
        row_start > hidden || row_count > hidden - row_start) return 0;
    float *a = (float *)malloc(sizeof(float) * (size_t)ffn);
    if (!a) return 0;
    double logit = 0.0;
    for (uint32_t i = 0; i < hidden; ++i) logit += (double)gate_inp[i] * x[i];
    const double sg = sigmoid_stable(logit);
    int ok = 1;
    for (uint32_t r = 0; r < ffn && ok; ++r) {
        double gd = 0.0, ud = 0.0;
        ok = dot_any(gate_up_type, gate + (size_t)r * grb, x, NULL, hidden, &gd) &&
             dot_any(gate_up_type, up + (size_t)r * grb, x, NULL, hidden, &ud);
        const float gf = (float)gd, uf = (float)ud;
        a[r] = (gf / (1.0f + expf(-gf))) * uf;
    }
    for (uint32_t i = 0; i < row_count && ok; ++i) {
        double v = 0.0;
        ok = dot_any(down_type, down + (size_t)(row_start + i) * drb, a, NULL, ffn, &v);
        out[i] = v * sg;
    }
    if (scalar) *scalar = sg;
    free(a);
    return ok;
}

/* native/redlite_native_engine_cpu.c:329-386 */
int orc_moe_layer(const orc_layer *L, const float *x, float *out, uint32_t *ids_out, float *weights_out, float *logits_out, int threads) {
    if (!L || !x || !out || !L->top_k || L->top_k > 64u || L->top_k > L->n_expert) return 0;
    const uint32_t H = L->hidden, F = L->ffn, E = L->n_expert, K = L->top_k;
    float *logits = (float *)malloc(sizeof(float) * ((size_t)E + H));
    double *routed = (double *)malloc(sizeof(double) * (size_t)H);
    uint32_t ids[64];
    float w[64];
    int ok = 0;
    if (!logits || !routed) goto out;
    float *sh = logits + E;
    if (!rows_mt(L->router_type, L->router, H, E, x, NULL, logits, NULL, threads)) goto out;
    if (!orc_router_select(logits, E, K, ids, w, NULL)) goto out;
    if (!routed_topk_mt(L->gate_up_type, L->down_type, L->gate, L->up, L->down,
                        F * orc_row_bytes(L->gate_up_type, H), F * orc_row_bytes(L->gate_up_type, H),
                        H * orc_row_bytes(L->down_type, F), ids, w, K, H, F, x, routed, threads)) goto out;
    double scalar = 0.0;
    if (!orc_shared_expert(L->sh_gate_up_type, L->sh_down_type, L->sh_gate, L->sh_up, L->sh_down, L->sh_gate_inp,
                           H, F, x, sh, &scalar, threads)) goto out;
    for (uint32_t i = 0; i < H; ++i) out[i] = (float)(routed[i] + (double)sh[i] * scalar);
    if (ids_out) memcpy(ids_out, ids, sizeof(uint32_t) * K);
    if (weights_out) memcpy(weights_out, w, sizeof(float) * K);
    if (logits_out) memcpy(logits_out, logits, sizeof(float) * E);
    ok = 1;
out:
    free(logits);
    free(routed);
    return ok;
}

int orc_moe_layer_batch(const orc_layer *L, const float *x, uint32_t ntok, float *out, uint32_t *ids, float *weights, int threads) {
    if (!L || !x || !out) return 0;
    for (uint32_t t = 0; t < ntok; ++t)
        if (!orc_moe_layer(L, x + (size_t)t * L->hidden, out + (size_t)t * L->hidden,
                           ids ? ids + (size_t)t * L->top_k : NULL, weights ? weights + (size_t)t * L->top_k : NULL, NULL, threads))
            return 0;
    return 1;
}

/* native/redmetal_engine_prefill.m:1246-1276 - union in first-appearance order, counting sort, stable placement */
int orc_group_pairs(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t n_expert,
                    uint32_t *uid, uint32_t *expert_start, uint32_t *pair_token, float *pair_weight, uint32_t *tok_pair) {
    if (!ids || !weights || !uid || !expert_start || !pair_token || !pair_weight || !tok_pair || !top_k || !n_expert) return -1;
    uint32_t *dense = (uint32_t *)malloc(sizeof(uint32_t) * 2u * (size_t)n_expert);
    if (!dense) return -1;
    uint32_t *cursor = dense + n_expert;
    for (uint32_t e = 0; e < n_expert; ++e) dense[e] = UINT32_MAX;
    uint32_t U = 0;
    for (uint32_t t = 0; t < ntok; ++t)
        for (uint32_t k = 0; k < top_k; ++k) {
            const uint32_t e = ids[(size_t)t * top_k + k];
            if (e >= n_expert) { free(dense); return -1; }
            if (dense[e] == UINT32_MAX) { dense[e] = U; uid[U++] = e; }
        }
    for (uint32_t u = 0; u <= U; ++u) expert_start[u] = 0;
    for (uint32_t i = 0; i < ntok * top_k; ++i) expert_start[dense[ids[i]] + 1u]++;
    for (uint32_t u = 0; u < U; ++u) expert_start[u + 1u] += expert_start[u];
    for (uint32_t u = 0; u < U; ++u) cursor[u] = expert_start[u];
    for (uint32_t t = 0; t < ntok; ++t)
        for (uint32_t k = 0; k < top_k; ++k) {
            const uint32_t p = cursor[dense[ids[(size_t)t * top_k + k]]]++;
            pair_token[p] = t;
            pair_weight[p] = weights[(size_t)t * top_k + k];
            tok_pair[(size_t)t * top_k + k] = p;
        }
    free(dense);
    return (int)U;
}
