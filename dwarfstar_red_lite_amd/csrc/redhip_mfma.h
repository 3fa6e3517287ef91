// Device helpers shared by the MFMA kernels on packed IQ2_XXS rows: fp16 hi/lo activation split, the LDS table of grid
// magnitudes, and the placement of the sign bits.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "redhip_decode.h"

namespace redhip {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// power-of-two pre-scale: largest |v| lands in [2^13, 2^14)
__device__ __forceinline__ int prescale_exp(float amax) {
    if (!(amax > 0.0f) || isinf(amax) || isnan(amax)) return 0;
    return (int)((__float_as_uint(amax) >> 23) & 255u) - 127 - 13;
}
__device__ __forceinline__ float exp2i(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }   // e in [-126, 127]

// v = hi + lo * 2^-11 (to 22 significant bits) after scaling by 2^-e
__device__ __forceinline__ void split_hi_lo(float v, float inv_scale, _Float16 *hi, _Float16 *lo) {
    const float t = v * inv_scale;
    const _Float16 h = (_Float16)t;
    *hi = h;
    *lo = (_Float16)((t - (float)h) * 2048.0f);
}


// block scale d of a packed row: one conversion instruction (fp16 subnormals are exact, a NaN stays a NaN)
__device__ __forceinline__ float scale_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }

constexpr int kWaves = 16;                      // 1024 lanes per gate/up workgroup
constexpr uint32_t kMagBytes = 256u * 16u;      // eight fp16 magnitudes per grid entry

// LDS decode table (eight fp16 magnitudes per grid entry), built by the first 256 lanes of a workgroup
__device__ __forceinline__ void build_tables(uint8_t *lds, uint32_t tid, uint64_t grid_entry) {
    if (tid < 256u) {
        uint32_t w4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const _Float16 lo = (_Float16)(float)((uint32_t)(grid_entry >> (16 * i)) & 255u), hi = (_Float16)(float)((uint32_t)(grid_entry >> (16 * i + 8)) & 255u);
            w4[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint4 *>(lds + (size_t)tid * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
}


// Eight signed fp16 weights of one grid entry: magnitudes from the LDS table, signs placed by integer arithmetic.
// s8 = s7 | parity << 7 holds one sign bit per weight; weight 2i sits in bits 0..15 of word i, weight 2i + 1 in
// bits 16..31, so word i needs bit 2i of s8 at bit 15 and bit 2i + 1 at bit 31: one 24-bit multiply by
// 2^(7 - 2i) + 2^(22 - 2i) of s8 << 8 puts both there (the two shifted copies do not overlap).
union WeightQuad { uint32_t u[2]; half4_t h; };
__device__ __forceinline__ void place_signs(uint4 m, uint32_t s7, WeightQuad &b0, WeightQuad &b1) {
    const uint32_t s8s = (s7 << 8) | ((__popc(s7) & 1u) << 15);
    b0.u[0] = (__umul24(s8s, (1u << 7) | (1u << 22)) & 0x80008000u) | m.x;
    b0.u[1] = (__umul24(s8s, (1u << 5) | (1u << 20)) & 0x80008000u) | m.y;
    b1.u[0] = (__umul24(s8s, (1u << 3) | (1u << 18)) & 0x80008000u) | m.z;
    b1.u[1] = (__umul24(s8s, (1u << 1) | (1u << 16)) & 0x80008000u) | m.w;
}
__device__ __forceinline__ void signed_weights(const uint8_t *lds, uint32_t idx, uint32_t s7, WeightQuad &b0, WeightQuad &b1) {
    place_signs(*reinterpret_cast<const uint4 *>(lds + (idx << 4)), s7, b0, b1);
}


// fp16 copy of a caller-supplied codebook (int8 [entries][8]) in LDS, 16 bytes per entry; built by `builders` lanes starting at lane `first`
// of the workgroup (the gate/up kernel: every wave but the first, which selects meanwhile)
template <int FMT>
__device__ __forceinline__ void build_codebook_table(uint8_t *lds, uint32_t tid, const int8_t *grid, uint32_t first = 64u, uint32_t builders = (kWaves - 1) * 64u) {
    constexpr uint32_t kEntries = FMT == 1 ? 512u : 2048u;
    for (uint32_t i = tid - first; i < kEntries; i += builders) {      // tid < first wraps past the bound
        const uint64_t e = reinterpret_cast<const uint64_t *>(grid)[i];
        uint32_t w4[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const _Float16 lo = (_Float16)(float)(int8_t)(e >> (16 * k)), hi = (_Float16)(float)(int8_t)(e >> (16 * k + 8));
            w4[k] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint4 *>(lds + (size_t)i * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
}
// The same table built by all 1024 lanes of a workgroup in two steps: codebook_seed requests a lane's entries (tid, and tid + 1024 for the
// 2048-entry codebook), build_codebook_table_from converts and stores them - for kernels that want the request in flight early.
template <int FMT>
__device__ __forceinline__ void codebook_seed(uint32_t tid, const int8_t *grid, uint64_t (&seed)[2]) {
    constexpr uint32_t kEntries = FMT == 1 ? 512u : 2048u;
    seed[0] = tid < kEntries ? reinterpret_cast<const uint64_t *>(grid)[tid] : 0ull;
    seed[1] = tid + 1024u < kEntries ? reinterpret_cast<const uint64_t *>(grid)[tid + 1024u] : 0ull;
}
template <int FMT>
__device__ __forceinline__ void build_codebook_table_from(uint8_t *lds, uint32_t tid, const uint64_t (&seed)[2]) {
    constexpr uint32_t kEntries = FMT == 1 ? 512u : 2048u;
#pragma unroll
    for (uint32_t r = 0; r < 2u; ++r) {
        const uint32_t i = tid + 1024u * r;
        if (i < kEntries) {
            const uint64_t e = seed[r];
            uint32_t w4[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const _Float16 lo = (_Float16)(float)(int8_t)(e >> (16 * k)), hi = (_Float16)(float)(int8_t)(e >> (16 * k + 8));
                w4[k] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
            }
            *reinterpret_cast<uint4 *>(lds + (size_t)i * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
        }
    }
}

}  // namespace redhip
