// Device-side decoders of the GGUF block formats on this path, straight from the raw block bytes.
// A "chunk" is 32 consecutive weights of a row (one IQ2_XXS group, one IQ3_S sub-block, a quarter of a Q6_K
// half); every format keeps one scale per chunk or per half chunk, so 32 is the natural unit of work per lane.
// All products below have at most 24 significant bits, so the f32 results do not depend on evaluation order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "redhip_internal.h"
#define REDHIP_TABLE_ATTR __device__
#include "redhip_tables.h"

namespace redhip {


__device__ __forceinline__ uint32_t ld_u16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t *p) {   // 4 bytes at a 2-byte aligned address
    return ld_u16(p) | (ld_u16(p + 2) << 16);
}

// IEEE binary16 bits -> f32, exact for every pattern (subnormals by integer scaling, NaN payload kept)
__device__ __forceinline__ float half_bits_to_f32(uint32_t h) {
    const uint32_t e = (h >> 10) & 31u, m = h & 1023u, s = (h & 0x8000u) << 16;
    uint32_t u;
    if (e == 0u) u = __float_as_uint((float)m * 5.9604644775390625e-8f) | s;      // m * 2^-24, exact
    else if (e == 31u) u = s | 0x7f800000u | (m << 13);
    else u = s | ((e + 112u) << 23) | (m << 13);
    return __uint_as_float(u);
}

__device__ __forceinline__ float apply_sign(float v, uint32_t negative) {
    return __uint_as_float(__float_as_uint(v) ^ (negative << 31));
}

template <uint32_t T> struct Fmt;
template <> struct Fmt<T_IQ2_XXS> { static constexpr uint32_t kBlock = 66u; };
template <> struct Fmt<T_IQ3_S> { static constexpr uint32_t kBlock = 110u; };
template <> struct Fmt<T_Q6_K> { static constexpr uint32_t kBlock = 210u; };
template <> struct Fmt<T_F32> { static constexpr uint32_t kBlock = 1024u; };   // 256 floats
template <> struct Fmt<T_IQ2_XS> { static constexpr uint32_t kBlock = 74u; };
template <> struct Fmt<T_IQ1_M> { static constexpr uint32_t kBlock = 56u; };
// bytes of the caller-supplied codebook a format decodes through (int8 [entries][8]); 0: the codebook is built in
template <uint32_t T> struct Codebook { static constexpr uint32_t kBytes = 0u; };
template <> struct Codebook<T_IQ2_XS> { static constexpr uint32_t kBytes = 512u * 8u; };
template <> struct Codebook<T_IQ1_M> { static constexpr uint32_t kBytes = 2048u * 8u; };

// w[0..32) = weights [32*chunk, 32*chunk + 32) of the row starting at `row`
template <uint32_t T> __device__ __forceinline__ void decode32(const uint8_t *row, uint32_t chunk, float *w);

template <> __device__ __forceinline__ void decode32<T_F32>(const uint8_t *row, uint32_t chunk, float *w) {
    const float4 *p = reinterpret_cast<const float4 *>(row) + 8u * chunk;
#pragma unroll
    for (int i = 0; i < 8; ++i) { const float4 v = p[i]; w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w; }
}

template <> __device__ __forceinline__ void decode32<T_IQ2_XXS>(const uint8_t *row, uint32_t chunk, float *w) {
    const uint8_t *bp = row + (size_t)(chunk >> 3) * 66u;
    const uint32_t g = chunk & 7u;
    const float d = half_bits_to_f32(ld_u16(bp));
    const uint32_t idx4 = ld_u32_a2(bp + 2u + 8u * g);
    const uint32_t aux = ld_u32_a2(bp + 6u + 8u * g);
    const float db = d * (0.5f + (float)(aux >> 28)) * 0.25f;
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint64_t mag = redhip_iq2xxs_grid[(idx4 >> (8u * l)) & 255u];
        const uint32_t s7 = (aux >> (7u * l)) & 127u;
        const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j)
            w[8u * l + j] = apply_sign(db * (float)((uint32_t)(mag >> (8u * j)) & 255u), (s8 >> j) & 1u);
    }
}

template <> __device__ __forceinline__ void decode32<T_IQ3_S>(const uint8_t *row, uint32_t chunk, float *w) {
    const uint8_t *bp = row + (size_t)(chunk >> 3) * 110u;
    const uint32_t sub = chunk & 7u;
    const float d = half_bits_to_f32(ld_u16(bp));
    const uint32_t nib = ((uint32_t)bp[106u + (sub >> 1)] >> (4u * (sub & 1u))) & 15u;
    const float db = d * (float)(1u + 2u * nib);
    const uint32_t qh = bp[66u + sub];
    const uint32_t qs_lo = ld_u32_a2(bp + 2u + 8u * sub), qs_hi = ld_u32_a2(bp + 6u + 8u * sub);
    const uint32_t sg4 = ld_u32_a2(bp + 74u + 4u * sub);
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t pair = (l < 2u ? qs_lo >> (16u * l) : qs_hi >> (16u * (l - 2u))) & 0xffffu;
        const uint32_t ia = (pair & 255u) | ((qh << (8u - 2u * l)) & 256u);
        const uint32_t ib = (pair >> 8) | ((qh << (7u - 2u * l)) & 256u);
        const uint32_t wa = redhip_iq3s_grid[ia], wb = redhip_iq3s_grid[ib];
        const uint32_t sg = (sg4 >> (8u * l)) & 255u;
#pragma unroll
        for (uint32_t j = 0; j < 4u; ++j) {
            w[8u * l + j] = apply_sign(db * (float)((wa >> (8u * j)) & 255u), (sg >> j) & 1u);
            w[8u * l + 4u + j] = apply_sign(db * (float)((wb >> (8u * j)) & 255u), (sg >> (4u + j)) & 1u);
        }
    }
}

template <> __device__ __forceinline__ void decode32<T_Q6_K>(const uint8_t *row, uint32_t chunk, float *w) {
    const uint8_t *bp = row + (size_t)(chunk >> 3) * 210u;
    const uint32_t sub = chunk & 7u, half = sub >> 2, q = sub & 3u;
    const float d = half_bits_to_f32(ld_u16(bp + 208u));
    const uint8_t *ql = bp + 64u * half + 32u * (q & 1u);     // q1,q3 read ql[l], q2,q4 read ql[l + 32]
    const uint8_t *qh = bp + 128u + 32u * half;
    const int8_t *sc = reinterpret_cast<const int8_t *>(bp + 192u + 8u * half + 2u * q);
    const float d0 = d * (float)sc[0], d1 = d * (float)sc[1];
#pragma unroll
    for (uint32_t i = 0; i < 16u; ++i) {                      // two weights per 16-bit load
        const uint32_t lo2 = ld_u16(ql + 2u * i), hi2 = ld_u16(qh + 2u * i);
#pragma unroll
        for (uint32_t b = 0; b < 2u; ++b) {
            const uint32_t lb = (lo2 >> (8u * b)) & 255u, hb = (hi2 >> (8u * b)) & 255u;
            const uint32_t nib = (q & 2u) ? (lb >> 4) : (lb & 15u);
            const int v = (int)(nib | (((hb >> (2u * q)) & 3u) << 4)) - 32;
            const uint32_t l = 2u * i + b;
            w[l] = (l < 16u ? d0 : d1) * (float)v;
        }
    }
}

// Formats that decode through a caller-supplied codebook: `grid` is that codebook, in global memory or a copy in LDS.
template <uint32_t T> __device__ __forceinline__ void decode32_cb(const uint8_t *row, uint32_t chunk, float *w, const int8_t *grid) {
    (void)grid;
    decode32<T>(row, chunk, w);
}

// IQ2_XS, native/redlite_native_reference.c:116-142: block = f16 d, 32 x u16 (9-bit codebook index + 7 sign bits, the
// eighth sign is their parity), 8 bytes of 4-bit scales (one per 16 weights); weight = d * (0.5 + scale) * 0.25 * entry * sign
template <> __device__ __forceinline__ void decode32_cb<T_IQ2_XS>(const uint8_t *row, uint32_t chunk, float *w, const int8_t *grid) {
    const uint8_t *bp = row + (size_t)(chunk >> 3) * 74u;
    const uint32_t cb = chunk & 7u;
    const float d = half_bits_to_f32(ld_u16(bp));
    const uint32_t sc = bp[66u + cb];
    const float db0 = d * (0.5f + (float)(sc & 15u)) * 0.25f, db1 = d * (0.5f + (float)(sc >> 4)) * 0.25f;
#pragma unroll
    for (uint32_t k = 0; k < 4u; ++k) {
        const uint32_t q = ld_u16(bp + 2u + 2u * (4u * cb + k));
        const int8_t *entry = grid + (q & 511u) * 8u;
        const uint32_t s7 = (q >> 9) & 127u, s8 = s7 | ((__popc(s7) & 1u) << 7);
        const float db = k < 2u ? db0 : db1;
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) w[8u * k + j] = apply_sign(db * (float)entry[j], (s8 >> j) & 1u);
    }
}

// IQ1_M, native/redlite_native_reference.c:149-170: block = 32 index bytes, 16 bytes of nibbles (3 high index bits + the
// sign of the 1/8 offset), four u16 with 3-bit scales (one per 16 weights) and the f16 d spread over their top nibbles;
// weight = d * (2 * scale + 1) * (entry + or - 0.125), entry in {-1, 0, 1}
template <> __device__ __forceinline__ void decode32_cb<T_IQ1_M>(const uint8_t *row, uint32_t chunk, float *w, const int8_t *grid) {
    const uint8_t *bp = row + (size_t)(chunk >> 3) * 56u;
    const uint32_t cb = chunk & 7u;
    uint32_t sc[4];
#pragma unroll
    for (uint32_t i = 0; i < 4u; ++i) sc[i] = ld_u16(bp + 48u + 2u * i);
    const float d = half_bits_to_f32((sc[0] >> 12) | ((sc[1] >> 8) & 0x00f0u) | ((sc[2] >> 4) & 0x0f00u) | (sc[3] & 0xf000u));
#pragma unroll
    for (uint32_t k = 0; k < 4u; ++k) {
        const uint32_t group = 4u * cb + k;
        const uint32_t nibble = ((uint32_t)bp[32u + (group >> 1)] >> (4u * (group & 1u))) & 15u;
        const int8_t *entry = grid + ((uint32_t)bp[group] | ((nibble & 7u) << 8)) * 8u;
        const float delta = (nibble & 8u) ? -0.125f : 0.125f;
        const uint32_t si = group >> 1;
        const float dl = d * (float)(2u * ((sc[si >> 2] >> (3u * (si & 3u))) & 7u) + 1u);
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) w[8u * k + j] = dl * ((float)entry[j] + delta);
    }
}

}  // namespace redhip
