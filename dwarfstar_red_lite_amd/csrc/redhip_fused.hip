// Kernels on packed IQ2_XXS rows for one token and for small batches; no atomics and no device-scope fences (on this
// hardware a grid-wide __threadfence costs tens of microseconds and same-address float atomics serialise), so kernel
// boundaries are the only grid-wide synchronisation.
//
// One token, three launches per layer:
//   router_*_kernel        logits of every expert (plus the shared expert's gate logit) and the fp16 split of x; for a
//                          Q6_K shared expert also its gate and up products, in extra workgroups
//   all matrices IQ2_XXS:
//   expert_slice_kernel    one workgroup per (slot, 32 ffn columns): softmax top-k on one wave, the slot's 32 gate + 32 up rows,
//                          SwiGLU, then the matching 32 columns of its down matrix (column-sliced copy), weighted -> a partial
//                          output vector per workgroup
//   slice_sum_kernel       the (top_k + 1) * ffn / 32 partial vectors added in a fixed order: deterministic
//   mixed layouts whose batches run as slices (IQ2_XXS gate / up with IQ3_S down, all IQ2_XS, all IQ1_M): the same two kernels, the
//   down slices from the column-sliced words / streams, the shared expert from dense f32 copies (its gate / up products by the router launch)
//   other mixed layouts:
//   gateup_select_kernel   the same selection, then 32 gate rows + 32 up rows of one selected expert -> SwiGLU -> fp16 halves
//   down_combine_*_kernel  8 output rows per workgroup, one wave per selected expert; weighted sum in selection order + shared
//                          expert * scalar gate (word-packed IQ3_S / stream-packed IQ2_XS, IQ1_M on the MFMA, other types raw rows)
// Small batches (two to 32 tokens behind the layer's own router, fewer with a caller's routing): pairs grouped by expert (group_small, in
// the first launch, with the selection in one of its own, or alone), then batch_slice_kernel + slice_sum_kernel (a pass = two tokens of one
// expert), or gateup_batch_kernel + down_batch_*_kernel (the other mixed layouts: persistent workgroups, every distinct expert read once).
//
// Arithmetic: a weight is (sign * magnitude * (2*scale+1)) * d/8; the eight magnitudes of a grid entry are exact fp16
// values from an LDS table, the sign bits are placed by integer arithmetic; an activation vector is split into two
// fp16 halves (hi + lo*2^-11, after a power-of-two pre-scale), and v_mfma_f32_4x4x4_16B_f16 multiplies four weights of
// four rows by both halves per lane with fp32 accumulation. Per-group scales and d are applied to the fp32 sums.
//
// Layout ("packed IQ2_XXS"): the 66-byte blocks are split at upload into an 8-byte stream [row][group] (4 grid
// indices + 28 sign bits + 4 scale bits per 32 weights) and an fp16 stream [row][block] (d per 256 weights), both
// naturally aligned. Same total bytes as the GGUF blocks.
#include <type_traits>
#include <hip/hip_fp16.h>

#include "redhip_decode.h"
#include "redhip_mfma.h"

namespace redhip {

// ---- in-kernel phase stamps (only in a library built with -DREDHIP_TIMELINE; the counterpart of the reference's RL_ENGINE_PROFILE for what
// happens inside one launch) ----
// REDHIP_STAMP(slot) in a kernel: lane 0 of the workgroup stores the 100 MHz wall clock into timeline[workgroup][slot] (workgroup = its
// linear index in the grid, the first kTimelineGroups of them; slot < kTimelineSlots; slot kTimelineSlots - 1 holds the compute unit the
// workgroup ran on, slots 13 and 14 the shader clock counter at stamps 3 and 4: with the wall clock of the same stamps, the clock rate).
// redhip_timeline_read copies the array out. Without the flag the macro is empty and the array does not exist.
[[maybe_unused]] constexpr uint32_t kTimelineGroups = 2048u, kTimelineSlots = 16u;
#if defined(REDHIP_TIMELINE) && defined(__HIPCC__)
__device__ unsigned long long g_timeline[kTimelineGroups * kTimelineSlots];      // (device symbols are private to a source file here: the stamps and their reader live in this one)
__device__ __forceinline__ void timeline_stamp(uint32_t slot) {
    if (threadIdx.x == 0u) {
        const uint32_t wg = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        if (wg < kTimelineGroups) {
            g_timeline[wg * kTimelineSlots + slot] = wall_clock64();
            if (slot == 0u) g_timeline[wg * kTimelineSlots + kTimelineSlots - 1u] = __smid();
            if (slot == 3u || slot == 4u) g_timeline[wg * kTimelineSlots + 10u + slot] = clock64();      // slots 13, 14: the shader clock around one phase
        }
    }
}
#define REDHIP_STAMP(slot) ::redhip::timeline_stamp(slot)
#else
#define REDHIP_STAMP(slot) do {} while (0)
#endif




// ---------------------------------------------------------------- repacking (upload time)

// raw rows [nrows][K/256 blocks of 66 B] -> qs [nrows][K/32] uint2, ds [nrows][K/256] u16      (col_major = 0)
//                                        -> qs [K/32][nrows] uint2, ds [K/256][nrows] u16      (col_major = 1)
__global__ void repack_iq2xxs_kernel(const uint8_t *raw0, uint64_t raw_stride, uint32_t nrows, uint32_t K, int col_major,
                                     uint8_t *packed0, uint64_t packed_stride) {
    const uint32_t groups = K / 32u, blocks = K / 256u;
    const uint8_t *raw = raw0 + (uint64_t)blockIdx.y * raw_stride;          // blockIdx.y = matrix of the batch
    uint2 *qs = reinterpret_cast<uint2 *>(packed0 + (uint64_t)blockIdx.y * packed_stride);
    uint16_t *ds = reinterpret_cast<uint16_t *>(packed0 + (uint64_t)blockIdx.y * packed_stride + (uint64_t)nrows * groups * 8u);
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * groups) return;
    const uint32_t r = (uint32_t)(gid / groups), g = (uint32_t)(gid % groups);
    const uint8_t *bp = raw + ((uint64_t)r * blocks + (g >> 3)) * 66u;
    const uint2 v = make_uint2(ld_u32_a2(bp + 2u + 8u * (g & 7u)), ld_u32_a2(bp + 6u + 8u * (g & 7u)));
    if (col_major) qs[(uint64_t)g * nrows + r] = v; else qs[(uint64_t)r * groups + g] = v;
    if ((g & 7u) == 0u) {
        const uint16_t d = (uint16_t)ld_u16(bp);
        if (col_major) ds[(uint64_t)(g >> 3) * nrows + r] = d; else ds[(uint64_t)r * blocks + (g >> 3)] = d;
    }
}

hipError_t launch_repack_iq2xxs(const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K, bool col_major,
                                void *packed, uint64_t packed_stride, hipStream_t s) {
    if (!nrows || !K || K % 256u || !count || count > 65535u) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    REDHIP_LAUNCH(repack_iq2xxs_kernel, dim3((uint32_t)((total + 255u) / 256u), count), dim3(256), 0, s,
                  static_cast<const uint8_t *>(raw), raw_stride, nrows, K, col_major ? 1 : 0, static_cast<uint8_t *>(packed), packed_stride);
    return hipGetLastError();
}

// The same split for the two formats that decode through caller-supplied codebooks (col_major as above: every array [group or block][row]):
//   IQ2_XS (74-byte blocks): qs [nrows][K/32] uint2 = the group's four u16 (9-bit index + 7 sign bits each), ds [nrows][K/256] u16,
//                            sc [nrows][K/32] u8 = the group's two 4-bit scales (one per 16 weights)
//   IQ1_M (56-byte blocks):  qs [nrows][K/32] uint2: x = the group's four low index bytes, y = its four nibbles (3 high index bits +
//                            offset sign) | scale of the first 16 weights << 16 | scale of the second 16 << 19; ds [nrows][K/256] u16 = d
//                            gathered from the top nibbles of the block's four scale words
template <uint32_t T>
__global__ void repack_codebook_kernel(const uint8_t *raw0, uint64_t raw_stride, uint32_t nrows, uint32_t K, int col_major, uint8_t *packed0, uint64_t packed_stride) {
    const uint32_t groups = K / 32u, blocks = K / 256u;
    const uint8_t *raw = raw0 + (uint64_t)blockIdx.y * raw_stride;
    uint8_t *pk = packed0 + (uint64_t)blockIdx.y * packed_stride;
    uint2 *qs = reinterpret_cast<uint2 *>(pk);
    uint16_t *ds = reinterpret_cast<uint16_t *>(pk + (uint64_t)nrows * groups * 8u);
    uint8_t *sc = pk + (uint64_t)nrows * groups * 8u + (uint64_t)nrows * blocks * 2u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * groups) return;
    const uint32_t r = (uint32_t)(gid / groups), g = (uint32_t)(gid % groups), gb = g & 7u;
    const uint8_t *bp = raw + ((uint64_t)r * blocks + (g >> 3)) * Fmt<T>::kBlock;
    const uint64_t at = col_major ? (uint64_t)g * nrows + r : gid, d_at = col_major ? (uint64_t)(g >> 3) * nrows + r : (uint64_t)r * blocks + (g >> 3);
    if constexpr (T == T_IQ2_XS) {
        qs[at] = make_uint2(ld_u32_a2(bp + 2u + 8u * gb), ld_u32_a2(bp + 6u + 8u * gb));
        sc[at] = bp[66u + gb];
        if (gb == 0u) ds[d_at] = (uint16_t)ld_u16(bp);
    } else {
        const uint32_t word = ld_u16(bp + 48u + 2u * (gb >> 1)), sh = 6u * (gb & 1u);
        qs[at] = make_uint2(ld_u32_a2(bp + 4u * gb), ld_u16(bp + 32u + 2u * gb) | (((word >> sh) & 7u) << 16) | (((word >> (sh + 3u)) & 7u) << 19));
        if (gb == 0u) {
            const uint32_t s0 = ld_u16(bp + 48u), s1 = ld_u16(bp + 50u), s2 = ld_u16(bp + 52u), s3 = ld_u16(bp + 54u);
            ds[d_at] = (uint16_t)((s0 >> 12) | ((s1 >> 8) & 0x00f0u) | ((s2 >> 4) & 0x0f00u) | (s3 & 0xf000u));
        }
    }
}

// gate / up matrices of `type` (IQ2_XXS, IQ2_XS, IQ1_M) into the streams the one-token gate/up kernel reads; packed_matrix_bytes() each
hipError_t launch_repack_gateup(uint32_t type, const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K,
                                void *packed, uint64_t packed_stride, hipStream_t s, bool col_major) {
    if (type == T_IQ2_XXS) return launch_repack_iq2xxs(raw, raw_stride, count, nrows, K, col_major, packed, packed_stride, s);
    if (!nrows || !K || K % 256u || !count || count > 65535u) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    const dim3 grid((uint32_t)((total + 255u) / 256u), count);
    if (type == T_IQ2_XS)
        REDHIP_LAUNCH(repack_codebook_kernel<T_IQ2_XS>, grid, dim3(256), 0, s, static_cast<const uint8_t *>(raw), raw_stride, nrows, K, col_major ? 1 : 0, static_cast<uint8_t *>(packed), packed_stride);
    else if (type == T_IQ1_M)
        REDHIP_LAUNCH(repack_codebook_kernel<T_IQ1_M>, grid, dim3(256), 0, s, static_cast<const uint8_t *>(raw), raw_stride, nrows, K, col_major ? 1 : 0, static_cast<uint8_t *>(packed), packed_stride);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

// parity tap: f32 dequantisation straight from the packed streams (row-major output [nrows][K])
__global__ void dequant_packed_iq2xxs_kernel(const uint2 *qs, const uint16_t *ds, uint32_t nrows, uint32_t K, int col_major, float *out) {
    const uint32_t groups = K / 32u, blocks = K / 256u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * groups) return;
    const uint32_t r = (uint32_t)(gid / groups), g = (uint32_t)(gid % groups);
    const uint2 v = col_major ? qs[(uint64_t)g * nrows + r] : qs[(uint64_t)r * groups + g];
    const uint32_t dbits = col_major ? ds[(uint64_t)(g >> 3) * nrows + r] : ds[(uint64_t)r * blocks + (g >> 3)];
    const float db = half_bits_to_f32(dbits) * (0.5f + (float)(v.y >> 28)) * 0.25f;
    float *o = out + (uint64_t)r * K + 32u * g;
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint64_t mag = redhip_iq2xxs_grid[(v.x >> (8u * l)) & 255u];
        const uint32_t s7 = (v.y >> (7u * l)) & 127u, s8 = s7 | ((__popc(s7) & 1u) << 7);
        for (uint32_t j = 0; j < 8u; ++j) o[8u * l + j] = apply_sign(db * (float)((uint32_t)(mag >> (8u * j)) & 255u), (s8 >> j) & 1u);
    }
}

hipError_t launch_dequant_packed_iq2xxs(const void *packed, uint32_t nrows, uint32_t K, bool col_major, float *out, hipStream_t s) {
    if (!nrows || !K || K % 256u) return hipErrorInvalidValue;
    const uint2 *qs = static_cast<const uint2 *>(packed);
    const uint16_t *ds = reinterpret_cast<const uint16_t *>(static_cast<const uint8_t *>(packed) + (uint64_t)nrows * (K / 32u) * 8u);
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    REDHIP_LAUNCH(dequant_packed_iq2xxs_kernel, dim3((uint32_t)((total + 255u) / 256u)), dim3(256), 0, s, qs, ds, nrows, K, col_major ? 1 : 0, out);
    return hipGetLastError();
}

// the same tap for the packed IQ2_XS / IQ1_M streams; arithmetic as decode32_cb
template <uint32_t T>
__global__ void dequant_packed_codebook_kernel(const uint8_t *pk, uint32_t nrows, uint32_t K, const int8_t *grid, float *out, int col_major) {
    const uint32_t groups = K / 32u, blocks = K / 256u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * groups) return;
    const uint32_t r = (uint32_t)(gid / groups), g = (uint32_t)(gid % groups);
    const uint64_t at = col_major ? (uint64_t)g * nrows + r : gid, d_at = col_major ? (uint64_t)(g >> 3) * nrows + r : (uint64_t)r * blocks + (g >> 3);
    const uint2 v = reinterpret_cast<const uint2 *>(pk)[at];
    const float d = half_bits_to_f32(reinterpret_cast<const uint16_t *>(pk + (uint64_t)nrows * groups * 8u)[d_at]);
    float *o = out + (uint64_t)r * K + 32u * g;
    if constexpr (T == T_IQ2_XS) {
        const uint32_t sc = (pk + (uint64_t)nrows * groups * 8u + (uint64_t)nrows * blocks * 2u)[at];
        for (uint32_t l = 0; l < 4u; ++l) {
            const uint32_t w16 = ((l < 2u ? v.x : v.y) >> (16u * (l & 1u))) & 0xffffu;
            const int8_t *entry = grid + (w16 & 511u) * 8u;
            const uint32_t s7 = w16 >> 9, s8 = s7 | ((__popc(s7) & 1u) << 7);
            const float db = d * (0.5f + (float)(l < 2u ? (sc & 15u) : (sc >> 4))) * 0.25f;
            for (uint32_t j = 0; j < 8u; ++j) o[8u * l + j] = apply_sign(db * (float)entry[j], (s8 >> j) & 1u);
        }
    } else {
        for (uint32_t l = 0; l < 4u; ++l) {
            const int8_t *entry = grid + (((v.x >> (8u * l)) & 255u) | (((v.y >> (4u * l)) & 7u) << 8)) * 8u;
            const float delta = ((v.y >> (4u * l + 3u)) & 1u) ? -0.125f : 0.125f;
            const float dl = d * (float)(2u * ((v.y >> (l < 2u ? 16u : 19u)) & 7u) + 1u);
            for (uint32_t j = 0; j < 8u; ++j) o[8u * l + j] = dl * ((float)entry[j] + delta);
        }
    }
}

hipError_t launch_dequant_packed(uint32_t type, const void *packed, uint32_t nrows, uint32_t K, const int8_t *grid, float *out, hipStream_t s, bool col_major) {
    if (type == T_IQ2_XXS) return launch_dequant_packed_iq2xxs(packed, nrows, K, col_major, out, s);
    if (!nrows || !K || K % 256u || !grid) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    const dim3 grid_dim((uint32_t)((total + 255u) / 256u));
    if (type == T_IQ2_XS) REDHIP_LAUNCH(dequant_packed_codebook_kernel<T_IQ2_XS>, grid_dim, dim3(256), 0, s, static_cast<const uint8_t *>(packed), nrows, K, grid, out, col_major ? 1 : 0);
    else if (type == T_IQ1_M) REDHIP_LAUNCH(dequant_packed_codebook_kernel<T_IQ1_M>, grid_dim, dim3(256), 0, s, static_cast<const uint8_t *>(packed), nrows, K, grid, out, col_major ? 1 : 0);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// ---------------------------------------------------------------- router GEMV + tail

// Wave-wide reductions without LDS traffic: quad permutes and row rotations (DPP) inside rows of 16 lanes, then
// swaps of odd/even rows and of the two halves of the wave. Every lane ends with the result.
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL> __device__ __forceinline__ double dpp_f64(double v) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = __builtin_amdgcn_update_dpp(0u, (uint32_t)b, CTRL, 0xf, 0xf, false);
    const uint32_t hi = __builtin_amdgcn_update_dpp(0u, (uint32_t)(b >> 32), CTRL, 0xf, 0xf, false);
    return __builtin_bit_cast(double, (uint64_t)lo | ((uint64_t)hi << 32));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppRor4 = 0x124, kDppRor8 = 0x128;   // quad_perm [1,0,3,2], [2,3,0,1]; row_ror
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<kDppXor1>(v);
    v += dpp_f32<kDppXor2>(v);
    v += dpp_f32<kDppRor4>(v);
    v += dpp_f32<kDppRor8>(v);
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f32<kDppXor1>(v));
    v = fmaxf(v, dpp_f32<kDppXor2>(v));
    v = fmaxf(v, dpp_f32<kDppRor4>(v));
    v = fmaxf(v, dpp_f32<kDppRor8>(v));
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ double swap_halves_add(double v, bool rows) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)b, hi = (uint32_t)(b >> 32);
    uint64_t x, y;
    if (rows) {
        const auto a = __builtin_amdgcn_permlane16_swap(lo, lo, false, false), c = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
        x = (uint64_t)a[0] | ((uint64_t)c[0] << 32); y = (uint64_t)a[1] | ((uint64_t)c[1] << 32);
    } else {
        const auto a = __builtin_amdgcn_permlane32_swap(lo, lo, false, false), c = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
        x = (uint64_t)a[0] | ((uint64_t)c[0] << 32); y = (uint64_t)a[1] | ((uint64_t)c[1] << 32);
    }
    return __builtin_bit_cast(double, x) + __builtin_bit_cast(double, y);
}
__device__ __forceinline__ double wave_sum_d(double v) {
    v += dpp_f64<kDppXor1>(v);
    v += dpp_f64<kDppXor2>(v);
    v += dpp_f64<kDppRor4>(v);
    v += dpp_f64<kDppRor8>(v);
    v = swap_halves_add(v, true);
    return swap_halves_add(v, false);
}
// LDS written by some lanes of a wave becomes readable by its other lanes (one wave, no workgroup barrier)
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// Workgroup barrier for data exchanged through LDS only: waits for this wave's LDS operations, not for its outstanding global loads
// (__syncthreads waits for those too, so a workgroup that has requested its weights would sit at the barrier until the last of them has
// arrived; with this one every wave goes on to its first weights as soon as THEY are there).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
__device__ __forceinline__ uint32_t wave_count(bool pred) { return (uint32_t)__popcll(__ballot(pred)); }
// Raw GGUF rows are decoded from LDS: a wave copies `bytes` (a multiple of 16, both addresses 16-byte aligned) with
// coalesced 16-byte loads, so the many one- and two-byte fields of a block never go to memory one by one.
__device__ __forceinline__ void wave_stage(uint8_t *dst, const uint8_t *src, uint32_t bytes, uint32_t lane) {
    if (((uint32_t)(uintptr_t)src | bytes) % 16u == 0u) {
        for (uint32_t i = lane; i < bytes / 16u; i += 64u) reinterpret_cast<uint4 *>(dst)[i] = reinterpret_cast<const uint4 *>(src)[i];
    } else {                                             // GGUF blocks are always a multiple of two bytes
        for (uint32_t i = lane; i < bytes / 2u; i += 64u) reinterpret_cast<uint16_t *>(dst)[i] = reinterpret_cast<const uint16_t *>(src)[i];
    }
}

// One chunk of 32 Q6_K weights against 32 activations held in registers; sx0 / sx1 are the sums of the first and the
// second 16 activations. The 6-bit quants are unpacked four at a time with byte-parallel integer operations and enter
// the FMAs as unsigned bytes; the offset of 32 comes back through the activation sums:
//   sum (q - 32) d s x = d s (sum q x - 32 sum x).  Layout as native/redlite_native_quant_cpu.c:130-153 reads it.
__device__ __forceinline__ float q6k_dot32(const uint8_t *row, uint32_t chunk, const float *xv, float sx0, float sx1) {
    const uint8_t *bp = row + (size_t)(chunk >> 3) * 210u;
    const uint32_t sub = chunk & 7u, half = sub >> 2, q = sub & 3u;
    const uint8_t *ql = bp + 64u * half + 32u * (q & 1u), *qh = bp + 128u + 32u * half;
    const uint32_t scs = ld_u16(bp + 192u + 8u * half + 2u * q);
    const float d = half_bits_to_f32(ld_u16(bp + 208u));
    const float s0 = (float)(int)(int8_t)(scs & 255u), s1 = (float)(int)(int8_t)(scs >> 8);
    const uint32_t nib_shift = (q >> 1) * 4u, hi_shift = 2u * q;
    float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
    for (uint32_t v = 0; v < 8u; ++v) {
        uint32_t lo4, hi4;                               // 2-byte aligned: odd blocks of a row start at 2 mod 4
        __builtin_memcpy(&lo4, __builtin_assume_aligned(ql + 4u * v, 2), 4);
        __builtin_memcpy(&hi4, __builtin_assume_aligned(qh + 4u * v, 2), 4);
        const uint32_t q4 = ((lo4 >> nib_shift) & 0x0f0f0f0fu) | (((hi4 >> hi_shift) & 0x03030303u) << 4);
        float &acc = v < 4u ? acc0 : acc1;
        acc = fmaf((float)(q4 & 255u), xv[4u * v], acc);
        acc = fmaf((float)((q4 >> 8) & 255u), xv[4u * v + 1u], acc);
        acc = fmaf((float)((q4 >> 16) & 255u), xv[4u * v + 2u], acc);
        acc = fmaf((float)(q4 >> 24), xv[4u * v + 3u], acc);
    }
    return d * (s0 * fmaf(-32.0f, sx0, acc0) + s1 * fmaf(-32.0f, sx1, acc1));
}

// ---------------------------------------------------------------- grouping of at most 128 (token, k) pairs by expert

// Same outputs as the host pair sort it replaces: groups in first-appearance order, pairs of a group in token order.
// A table in LDS holds, per expert, the set of tokens that selected it (a token selects an expert at most once): the
// position of a pair inside its group and the group's size are bit counts of that set, the order of the groups a
// bit count over the "first pair of its expert" flags, the group offsets one prefix sum. Run by a whole workgroup
// of at least 256 threads (every thread reaches the barriers); one pair per lane of the first four waves - 256 pairs - or, in a workgroup
// of at least 512 threads, of the first eight - 512 pairs; at most 32 tokens (a token set is one word), 1024 experts.
constexpr uint32_t kGroupLdsWords = 1024u + 24u;
constexpr uint32_t kGroupSmallPairs = 256u, kGroupMaxPairs = 512u;
// Optionally also the pass list of the batched expert-slice kernel (g.pass_list != nullptr): a pass = up to two consecutive pairs of one
// group. Entry v: x = expert | pairs in the pass << 16; y = four bytes: the place k of the expert in the selection of its first and of
// its second pair's token, then the two tokens. Passes follow the groups' order; *g.n_pass = their number.
template <class PairId, class PairWeight>
__device__ __forceinline__ void group_small(const GroupJob &g, uint32_t *lds, PairId pair_id, PairWeight pair_w) {
    uint32_t *token_set = lds;                           // per expert: bit t = token t selected it; later the group's offset (| its first pass << 16)
    uint32_t *first_count = lds + 1024, *size_total = lds + 1032, *pass_total = lds + 1040;      // per wave of pairs (four or eight)
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u, K = g.top_k;
    const uint32_t npw = g.ntok * K > kGroupSmallPairs && blockDim.x >= 512u ? 8u : 4u;          // waves that hold pairs
    for (uint32_t i = tid; i < g.n_expert; i += blockDim.x) token_set[i] = 0u;
    __syncthreads();
    const uint32_t P = g.ntok * K, pr = tid;             // pair index (waves 0 .. npw - 1)
    const bool live = pr < P;
    const uint32_t t = live ? pr / K : 0u;
    const uint32_t e = live ? guarded_id(pair_id(t, pr % K), g.n_expert, g.status) : 0u;
    // A token that names an expert twice breaks the caller's contract: reported, and the repeated pair takes no place of its own in the
    // group arrays (it shares its twin's position, so every index stays inside the arrays of ntok * top_k pairs; expert_start[U] is then
    // the number of pairs placed, less than ntok * top_k)
    const bool dup = live && (atomicOr(&token_set[e], 1u << t) & (1u << t)) != 0u;
    if (dup && g.status) atomicOr(g.status, 2u);
    __syncthreads();
    const uint32_t set = live ? token_set[e] : 0u;
    const uint32_t n = (uint32_t)__popc(set), before = (uint32_t)__popc(set & ((1u << t) - 1u));
    const bool first = live && !dup && before == 0u;
    uint32_t scan = first ? n : 0u;                      // inclusive prefix sum of the group sizes in pair order
    const uint32_t n_pass_mine = first ? (n + 1u) >> 1 : 0u;
    uint32_t pscan = n_pass_mine;                        // the same of the groups' pass counts
    if (wave < npw) {
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = __shfl_up(scan, o, 64), pup = __shfl_up(pscan, o, 64);
            if (lane >= (uint32_t)o) { scan += up; pscan += pup; }
        }
        const uint64_t fm = __ballot(first);
        if (lane == 63u) { first_count[wave] = (uint32_t)__popcll(fm); size_total[wave] = scan; pass_total[wave] = pscan; }
    }
    const uint64_t first_mask = __ballot(first);
    __syncthreads();
    uint32_t groups_before = 0u, size_before = 0u, pass_before = 0u;      // totals of the waves of pairs before this one
#pragma unroll
    for (uint32_t w = 0; w < 7u; ++w)
        if (w < wave && wave < npw) { groups_before += first_count[w]; size_before += size_total[w]; pass_before += pass_total[w]; }
    const uint32_t grp = groups_before + __builtin_amdgcn_mbcnt_hi((uint32_t)(first_mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)first_mask, 0u));
    const uint32_t start = size_before + scan - (first ? n : 0u);
    const uint32_t pass0 = pass_before + pscan - n_pass_mine;
    if (first) { token_set[e] = start | (pass0 << 16); g.uid[grp] = e; g.expert_start[grp] = start; }
    if (tid == 0u) {
        uint32_t U = 0u, placed = 0u, passes = 0u;
        for (uint32_t w = 0; w < npw; ++w) { U += first_count[w]; placed += size_total[w]; passes += pass_total[w]; }
        g.expert_start[U] = placed;                      // = P unless a token repeated an expert
        g.n_unique[0] = U;
        if (g.n_pass) g.n_pass[0] = passes;
    }
    __syncthreads();
    if (live) {
        const uint32_t word = token_set[e], pos = (word & 0xffffu) + before;
        g.tok_pair[pr] = pos;
        if (!dup) {
            g.pair_token[pos] = t;
            g.pair_weight[pos] = pair_w(t, pr % K);
        }
        if (g.pass_list && !dup) {
            const uint32_t v = (word >> 16) + (before >> 1), half = before & 1u;
            uint8_t *entry = reinterpret_cast<uint8_t *>(g.pass_list + v);
            if (half == 0u) reinterpret_cast<uint32_t *>(entry)[0] = e | ((n - before >= 2u ? 2u : 1u) << 16);
            entry[4u + half] = (uint8_t)(pr % K);
            entry[6u + half] = (uint8_t)t;
        }
    }
}
// the same from routing held in device memory (kernels that carry the grouping as a side job of one extra workgroup)
__device__ __forceinline__ void group_small_given(const GroupJob &g, uint32_t *lds) {
    group_small(g, lds, [&](uint32_t t, uint32_t k) { return g.ids[t * g.top_k + k]; }, [&](uint32_t t, uint32_t k) { return g.weights[t * g.top_k + k]; });
}
__host__ inline bool group_job_fits(const GroupJob &g) {
    return g.ids && g.weights && g.ntok && g.ntok <= 16u && g.top_k && g.top_k <= 16u && g.ntok * g.top_k <= kGroupSmallPairs && g.n_expert && g.n_expert <= 1024u;
}

// ---------------------------------------------------------------- router GEMV

struct RouterArgs {
    const float *x;            // [ntok][hidden]
    const float *gate_inp;     // [hidden]
    float *logits;             // [ntok][n_expert + 1]; the extra entry is gate_inp . x (shared expert's gate logit)
    _Float16 *xh, *xl;         // [ntok][hidden] fp16 halves of x * 2^-xexp
    int *xexp;                 // [ntok]
    uint32_t hidden, n_expert;
    // Q6_K shared expert of a mixed-precision layout (single token): its gate and up rows (2 * ffn rows, the up matrix
    // right behind the gate matrix) are multiplied here, by workgroups behind the router's, into sh_gu [2 * ffn]
    const uint8_t *sh_q6k;
    const float *sh_dense;     // or the same 2 * ffn rows as f32 [2 * ffn][hidden] (f32 router kernel): rows behind the gate vector's
    float *sh_gu;
    uint32_t ffn;
    // block step: the activations are (x + branch) * rsqrt(mean((x + branch)^2) + eps) * norm_w, written to xn_out
    const float *branch, *norm_w;
    float eps;
    float *xn_out;             // [ntok][hidden]
    float *scalar_out;         // optional [ntok]: sigmoid of the gate logit (row n_expert), for callers that bring their own routing
};

// fp16 split of x, spread over the whole grid (every workgroup knows the largest |x| of its token)
__device__ __forceinline__ void split_x_job(const RouterArgs &a, uint32_t tok, float amax, float norm_inv, uint32_t n_blocks) {
    const uint32_t gt = blockIdx.x * blockDim.x + threadIdx.x, nt = n_blocks * blockDim.x;
    const int e = prescale_exp(amax);
    const float inv = exp2i(-e);
    const uint64_t base = (uint64_t)tok * a.hidden;
    for (uint32_t i = gt; i < a.hidden; i += nt) {
        float v = a.x[base + i];
        if (a.branch) {                                    // same expression as in the kernels: ((x + branch) * inv) * w
            v = ((v + a.branch[base + i]) * norm_inv) * a.norm_w[i];
            a.xn_out[base + i] = v;
        }
        split_hi_lo(v, inv, a.xh + base + i, a.xl + base + i);
    }
    if (gt == 0u) a.xexp[tok] = e;
}
// 1 / sqrt(mean of squares + eps) from a wave's (or workgroup's) sum of squares
__device__ __forceinline__ float norm_scale(double ss, uint32_t n, float eps) { return (float)(1.0 / sqrt(ss / (double)n + (double)eps)); }

// F32 router: one wave per row (row n_expert is the shared expert's gate vector), the row and x read as float4
// with lanes interleaved; every wave sees all of x, so the pre-scale exponent needs no extra pass. blockIdx.y = token.
template <int NV, int WPB = 4>          // float4 per lane: hidden = 256 * NV; WPB waves (rows) per workgroup
__global__ __launch_bounds__(WPB * 64) void router_f32_kernel(const float *w, const float *x_first, uint32_t hidden_first, uint32_t n_expert_first, RouterArgs a) {
    // (x_first, hidden_first, n_expert_first repeat a.x, a.hidden, a.n_expert: leading scalar arguments can reach a wave in registers at
    // its start, so the requests for the activations and for a router row leave before the argument block has come from memory)
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u, H = hidden_first, tok = blockIdx.y;
    const uint32_t r = blockIdx.x * WPB + wave;
    const float4 *xv = reinterpret_cast<const float4 *>(x_first + (uint64_t)tok * H);
    float4 wv[NV], xq[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) xq[k] = xv[lane + 64u * k];
    if (r < n_expert_first) {
        const float4 *wr = reinterpret_cast<const float4 *>(w + (uint64_t)r * H);
#pragma unroll
        for (int k = 0; k < NV; ++k) wv[k] = wr[lane + 64u * k];
    }
    const uint32_t n_rows = a.n_expert + 1u + (a.sh_dense ? 2u * a.ffn : 0u);      // router rows, the gate vector, then the shared expert's gate | up rows
    if (r >= a.n_expert && r < n_rows) {
        const float4 *wr = reinterpret_cast<const float4 *>(r == a.n_expert ? a.gate_inp : a.sh_dense + (uint64_t)(r - a.n_expert - 1u) * H);
#pragma unroll
        for (int k = 0; k < NV; ++k) wv[k] = wr[lane + 64u * k];
    }
    float norm_inv = 1.0f;
    if (a.branch) {                                        // every wave holds the whole vector: the norm needs no workgroup barrier
        const float4 *bv = reinterpret_cast<const float4 *>(a.branch + (uint64_t)tok * H), *nw = reinterpret_cast<const float4 *>(a.norm_w);
        float4 wn[NV];
        double ss = 0.0;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const float4 b = bv[lane + 64u * k];
            wn[k] = nw[lane + 64u * k];
            xq[k].x += b.x; xq[k].y += b.y; xq[k].z += b.z; xq[k].w += b.w;
            ss += ((double)xq[k].x * xq[k].x + (double)xq[k].y * xq[k].y) + ((double)xq[k].z * xq[k].z + (double)xq[k].w * xq[k].w);
        }
        norm_inv = norm_scale(wave_sum_d(ss), H, a.eps);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            xq[k].x = (xq[k].x * norm_inv) * wn[k].x; xq[k].y = (xq[k].y * norm_inv) * wn[k].y;
            xq[k].z = (xq[k].z * norm_inv) * wn[k].z; xq[k].w = (xq[k].w * norm_inv) * wn[k].w;
        }
    }
    float acc = 0.0f, amax = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        amax = fmaxf(fmaxf(amax, fmaxf(fabsf(xq[k].x), fabsf(xq[k].y))), fmaxf(fabsf(xq[k].z), fabsf(xq[k].w)));
        if (r < n_rows) {
            acc = fmaf(wv[k].x, xq[k].x, acc); acc = fmaf(wv[k].y, xq[k].y, acc);
            acc = fmaf(wv[k].z, xq[k].z, acc); acc = fmaf(wv[k].w, xq[k].w, acc);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0u && r <= a.n_expert) a.logits[(uint64_t)tok * (a.n_expert + 1u) + r] = acc;
    else if (lane == 0u && r < n_rows) a.sh_gu[(uint64_t)tok * 2u * a.ffn + (r - a.n_expert - 1u)] = acc;
    if (lane == 0u && r == a.n_expert && a.scalar_out) a.scalar_out[tok] = 1.0f / (1.0f + expf(-acc));      // as the selection computes it
    split_x_job(a, tok, wave_max(amax), norm_inv, gridDim.x);
}

// The same product for 2..8 tokens at once: a wave keeps its row in registers and walks the tokens, whose activation vectors (after the
// optional residual + norm, done by wave t for token t) sit in LDS, so a row is read once per batch instead of once per token.
template <int NV, int NWV>          // NWV waves (rows) per workgroup
__global__ __launch_bounds__(NWV * 64) void router_f32_multi_kernel(const float *w, const float *x_first, const float *gate_inp_first, const float *sh_dense_first, uint32_t hidden_first,
                                                                  uint32_t n_expert_first, uint32_t ffn_first, uint32_t ntok, uint32_t n_blocks, RouterArgs a, GroupJob job) {
    // (the leading arguments repeat a.x, a.gate_inp, a.sh_dense, a.hidden, a.n_expert, a.ffn; n_blocks = the workgroups that multiply rows:
    // leading scalar arguments can reach a wave in registers at its start, so the requests for its row and the activations leave at once)
    extern __shared__ __attribute__((aligned(16))) float xs_all[];      // [ntok][hidden]
    __shared__ float s_amax[16];
    if (blockIdx.x == n_blocks) {                        // the extra workgroup: pair sort of the caller's routing
        group_small_given(job, reinterpret_cast<uint32_t *>(xs_all));
        return;
    }
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u, H = hidden_first;
    const uint32_t r = blockIdx.x * (uint32_t)NWV + wave;
    const uint32_t n_rows = n_expert_first + 1u + (sh_dense_first ? 2u * ffn_first : 0u);
    const float4 *wr = reinterpret_cast<const float4 *>(r < n_expert_first ? w + (uint64_t)r * H : r == n_expert_first ? gate_inp_first
                                                        : sh_dense_first + (uint64_t)(r < n_rows ? r - n_expert_first - 1u : 0u) * H);
    float4 wv[NV];
    if (r < n_rows) {
#pragma unroll
        for (int k = 0; k < NV; ++k) wv[k] = wr[lane + 64u * k];
    }
    for (uint32_t tok = wave; tok < ntok; tok += (uint32_t)NWV) {
        const float4 *xv = reinterpret_cast<const float4 *>(x_first + (uint64_t)tok * H);
        float4 xq[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) xq[k] = xv[lane + 64u * k];
        float norm_inv = 1.0f;
        if (a.branch) {
            const float4 *bv = reinterpret_cast<const float4 *>(a.branch + (uint64_t)tok * H), *nw = reinterpret_cast<const float4 *>(a.norm_w);
            float4 wn[NV];
            double ss = 0.0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const float4 b = bv[lane + 64u * k];
                wn[k] = nw[lane + 64u * k];
                xq[k].x += b.x; xq[k].y += b.y; xq[k].z += b.z; xq[k].w += b.w;
                ss += ((double)xq[k].x * xq[k].x + (double)xq[k].y * xq[k].y) + ((double)xq[k].z * xq[k].z + (double)xq[k].w * xq[k].w);
            }
            norm_inv = norm_scale(wave_sum_d(ss), H, a.eps);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                xq[k].x = (xq[k].x * norm_inv) * wn[k].x; xq[k].y = (xq[k].y * norm_inv) * wn[k].y;
                xq[k].z = (xq[k].z * norm_inv) * wn[k].z; xq[k].w = (xq[k].w * norm_inv) * wn[k].w;
            }
        }
        float amax = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            amax = fmaxf(fmaxf(amax, fmaxf(fabsf(xq[k].x), fabsf(xq[k].y))), fmaxf(fabsf(xq[k].z), fabsf(xq[k].w)));
            reinterpret_cast<float4 *>(xs_all + (uint64_t)tok * H)[lane + 64u * k] = xq[k];
        }
        amax = wave_max(amax);
        if (lane == 0u) s_amax[tok] = amax;
    }
    __syncthreads();
    // fp16 split of all tokens, one element per thread over the first workgroups, from the copy in LDS (the values the products use)
    for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < ntok * H; idx += n_blocks * blockDim.x) {
        const uint32_t tok = idx / H;
        const float v = xs_all[idx];
        if (a.branch) a.xn_out[idx] = v;
        split_hi_lo(v, exp2i(-prescale_exp(s_amax[tok])), a.xh + idx, a.xl + idx);
        if (idx == tok * H) a.xexp[tok] = prescale_exp(s_amax[tok]);
    }
    for (uint32_t tok = 0; tok < ntok; ++tok) {
        const float4 *xq = reinterpret_cast<const float4 *>(xs_all + (uint64_t)tok * H);
        float acc = 0.0f;
        if (r < n_rows) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const float4 x4 = xq[lane + 64u * k];
                acc = fmaf(wv[k].x, x4.x, acc); acc = fmaf(wv[k].y, x4.y, acc);
                acc = fmaf(wv[k].z, x4.z, acc); acc = fmaf(wv[k].w, x4.w, acc);
            }
        }
        acc = wave_sum(acc);
        if (lane == 0u && r <= a.n_expert) a.logits[(uint64_t)tok * (a.n_expert + 1u) + r] = acc;
        else if (lane == 0u && r < n_rows) a.sh_gu[(uint64_t)tok * 2u * a.ffn + (r - a.n_expert - 1u)] = acc;
        if (lane == 0u && r == a.n_expert && a.scalar_out) a.scalar_out[tok] = 1.0f / (1.0f + expf(-acc));      // as the selection computes it
    }
}

// quantised router: rows decoded 32 weights per lane from the raw blocks, x staged in LDS
template <uint32_t T>
__global__ __launch_bounds__(256) void router_quant_kernel(const uint8_t *w, RouterArgs a) {
    __shared__ float lds_amax[4];
    __shared__ double lds_ss[4];
    extern __shared__ float xs[];                        // x (padded), then the four raw rows of the workgroup
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u, H = a.hidden, tok = blockIdx.y;
    const uint32_t row_bytes = (H / 256u) * Fmt<T>::kBlock;
    const uint32_t n_router_wg = (a.n_expert + 1u + 3u) / 4u;
    const bool shared_wg = blockIdx.x >= n_router_wg;                   // only launched when a.sh_q6k is set
    const uint32_t sh_row_bytes = (H / 256u) * 210u, sh_row0 = 8u * (blockIdx.x - n_router_wg) + 2u * wave;
    uint8_t *my_row = reinterpret_cast<uint8_t *>(xs + H + H / 32u) + wave * (shared_wg ? 2u * sh_row_bytes : ((row_bytes + 15u) & ~15u));
    if (shared_wg) wave_stage(my_row, a.sh_q6k + (uint64_t)sh_row0 * sh_row_bytes, 2u * sh_row_bytes, lane);      // the wave's two rows
    else if (blockIdx.x * 4u + wave < a.n_expert) wave_stage(my_row, w + (uint64_t)(blockIdx.x * 4u + wave) * row_bytes, row_bytes, lane);
    const float *x = a.x + (uint64_t)tok * H;
    float amax = 0.0f, norm_inv = 1.0f;
    if (a.branch) {                                      // two passes over the staged vector: sum of squares, then scale
        const float *br = a.branch + (uint64_t)tok * H;
        double ss = 0.0;
        for (uint32_t i = threadIdx.x; i < H; i += 256u) { const float v = x[i] + br[i]; xs[i + (i >> 5)] = v; ss += (double)v * v; }
        ss = wave_sum_d(ss);
        if (lane == 0u) lds_ss[wave] = ss;
        __syncthreads();
        norm_inv = norm_scale((lds_ss[0] + lds_ss[1]) + (lds_ss[2] + lds_ss[3]), H, a.eps);
        for (uint32_t i = threadIdx.x; i < H; i += 256u) { const float v = (xs[i + (i >> 5)] * norm_inv) * a.norm_w[i]; xs[i + (i >> 5)] = v; amax = fmaxf(amax, fabsf(v)); }
    } else {
        for (uint32_t i = threadIdx.x; i < H; i += 256u) { const float v = x[i]; xs[i + (i >> 5)] = v; amax = fmaxf(amax, fabsf(v)); }
    }
    amax = wave_max(amax);
    if (lane == 0u) lds_amax[wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(lds_amax[0], lds_amax[1]), fmaxf(lds_amax[2], lds_amax[3]));
    const uint32_t r = blockIdx.x * 4u + wave;
    if (shared_wg) {
        // 32 lanes per row, every 32nd chunk of 32 columns; the halves of the wave then add up separately
        const uint8_t *row = my_row + (lane >> 5) * sh_row_bytes;
        float acc = 0.0f;
        for (uint32_t c = lane & 31u; c < H / 32u; c += 32u) {
            float xv[32], sx0 = 0.0f, sx1 = 0.0f;
#pragma unroll
            for (int j = 0; j < 32; ++j) { xv[j] = xs[33u * c + j]; if (j < 16) sx0 += xv[j]; else sx1 += xv[j]; }
            acc += q6k_dot32(row, c, xv, sx0, sx1);
        }
        acc += dpp_f32<kDppXor1>(acc);
        acc += dpp_f32<kDppXor2>(acc);
        acc += dpp_f32<kDppRor4>(acc);
        acc += dpp_f32<kDppRor8>(acc);
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(acc), __float_as_uint(acc), false, false);
        acc = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);           // rows of 16 lanes: 0 + 1 and 2 + 3
        if ((lane & 31u) == 0u) a.sh_gu[(uint64_t)tok * 2u * a.ffn + sh_row0 + (lane >> 5)] = acc;
    } else if (r <= a.n_expert) {
        float acc = 0.0f;
        if (r < a.n_expert) {
            for (uint32_t c = lane; c < H / 32u; c += 64u) {
                if constexpr (T == T_Q6_K) {
                    float xv[32], sx0 = 0.0f, sx1 = 0.0f;
#pragma unroll
                    for (int j = 0; j < 32; ++j) { xv[j] = xs[33u * c + j]; if (j < 16) sx0 += xv[j]; else sx1 += xv[j]; }
                    acc += q6k_dot32(my_row, c, xv, sx0, sx1);
                } else {
                    float wv[32];
                    decode32<T>(my_row, c, wv);
                    float s = 0.0f;
#pragma unroll
                    for (int j = 0; j < 32; ++j) s = fmaf(wv[j], xs[33u * c + j], s);
                    acc += s;
                }
            }
        } else {
            const float4 *gp = reinterpret_cast<const float4 *>(a.gate_inp);
            for (uint32_t i0 = 0; i0 < H / 4u; i0 += 256u) {              // four float4 per lane in flight
                float4 gv[4];
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) { const uint32_t i = i0 + 64u * k + lane; gv[k] = i < H / 4u ? gp[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f); }
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) {
                    const uint32_t i = 4u * (i0 + 64u * k + lane);
                    if (i < H) {
                        const float *xp = xs + i + (i >> 5);
                        acc = fmaf(gv[k].x, xp[0], acc); acc = fmaf(gv[k].y, xp[1], acc); acc = fmaf(gv[k].z, xp[2], acc); acc = fmaf(gv[k].w, xp[3], acc);
                    }
                }
            }
        }
        acc = wave_sum(acc);
        if (lane == 0u) a.logits[(uint64_t)tok * (a.n_expert + 1u) + r] = acc;
    }
    split_x_job(a, tok, amax, norm_inv, gridDim.x);
}

hipError_t launch_router_gemv(uint32_t router_type, const void *w, const float *x, const float *gate_inp, uint32_t ntok, uint32_t hidden,
                              uint32_t n_expert, float *logits, void *xh, void *xl, int *xexp, const void *sh_q6k, float *sh_gu, uint32_t ffn,
                              hipStream_t s, const float *sh_dense, float *scalar_out, const GroupJob *job, bool *job_done) {
    if (!ntok || !hidden || hidden % 256u || (!n_expert && !sh_dense) || n_expert > 1024u) return hipErrorInvalidValue;      // n_expert 0: only the shared expert's rows
    const bool with_shared = sh_q6k && sh_gu && router_type == T_Q6_K && ntok <= 8u && ffn % 4u == 0u;      // sh_gu: [ntok][2 * ffn]
    const BlockContext &bc = block_context();
    if (bc.branch && (!bc.norm_w || !bc.xn_out)) return hipErrorInvalidValue;
    const bool with_dense = sh_dense && sh_gu && router_type == T_F32 && ntok <= 16u;      // sh_gu: [ntok][2 * ffn]
    if (job_done) *job_done = false;
    RouterArgs a{x, gate_inp, logits, static_cast<_Float16 *>(xh), static_cast<_Float16 *>(xl), xexp, hidden, n_expert,
                 with_shared ? static_cast<const uint8_t *>(sh_q6k) : nullptr, with_dense ? sh_dense : nullptr, sh_gu, ffn, bc.branch, bc.norm_w, bc.eps,
                 bc.xn_out, scalar_out};
    const dim3 grid((n_expert + 1u + (with_dense ? 2u * ffn : 0u) + 3u) / 4u, ntok);
    // F32 rows: a multiple of eight workgroups per token. Workgroups go to the eight XCDs in turn, so a row block then lands on the same
    // XCD for every token of the batch and all tokens but the first find it in that XCD's L2 instead of fetching the rows once per XCD.
    const dim3 grid8((grid.x + 7u) & ~7u, ntok);
    // with the shared expert's rows behind the router's (1537 rows at the benchmark shape) a row is read once for the whole batch; the
    // router's own 513 rows are quicker one token per grid layer (their re-reads hit the L2)
    if (router_type == T_F32 && with_dense && ntok >= 2u && (size_t)ntok * hidden * 4u <= 128u * 1024u) {
        const float *wf = static_cast<const float *>(w);
        const bool with_job = job && job_done && group_job_fits(*job);
        const dim3 mgrid((n_expert + 1u + 2u * ffn + 7u) / 8u + (with_job ? 1u : 0u));
        size_t lds = (size_t)ntok * hidden * 4u;
        if (with_job && lds < kGroupLdsWords * 4u) lds = kGroupLdsWords * 4u;
        const GroupJob gj = with_job ? *job : GroupJob{};
        // (64 KB of activations at 8 tokens of 2048, 128 KB at 16, beside a few static bytes: the limit is raised explicitly)
#define REDHIP_RMULTI(NV)                                                                                                                                  \
    do {                                                                                                                                                   \
        static bool attr = false;                                                                                                                           \
        if (!attr) {                                                                                                                                        \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(router_f32_multi_kernel<NV, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024); \
            if (e != hipSuccess) return e;                                                                                                                  \
            attr = true;                                                                                                                                    \
        }                                                                                                                                                   \
        REDHIP_LAUNCH((router_f32_multi_kernel<NV, 8>), mgrid, dim3(512), lds, s, wf, a.x, a.gate_inp, a.sh_dense, a.hidden, a.n_expert, a.ffn, ntok,       \
                      mgrid.x - (gj.ids ? 1u : 0u), a, gj);                                                                                                 \
        if (with_job) *job_done = true;                                                                                                                     \
        return hipGetLastError();                                                                                                                           \
    } while (0)
        switch (hidden / 256u) {
            case 2: REDHIP_RMULTI(2);
            case 4: REDHIP_RMULTI(4);
            case 8: REDHIP_RMULTI(8);
            default: break;
        }
#undef REDHIP_RMULTI
    }
    if (router_type == T_F32) {
        const float *wf = static_cast<const float *>(w);
        switch (hidden / 256u) {
            case 2: REDHIP_LAUNCH(router_f32_kernel<2>, grid8, dim3(256), 0, s, wf, a.x, a.hidden, a.n_expert, a); break;
            case 4: REDHIP_LAUNCH(router_f32_kernel<4>, grid8, dim3(256), 0, s, wf, a.x, a.hidden, a.n_expert, a); break;
            case 8: REDHIP_LAUNCH(router_f32_kernel<8>, grid8, dim3(256), 0, s, wf, a.x, a.hidden, a.n_expert, a); break;      // (one or two rows per workgroup instead of four: no difference)
            case 16: REDHIP_LAUNCH(router_f32_kernel<16>, grid8, dim3(256), 0, s, wf, a.x, a.hidden, a.n_expert, a); break;
            default: return hipErrorInvalidValue;
        }
    } else if (router_type == T_Q6_K) {
        const size_t lds = (size_t)(hidden + hidden / 32u) * sizeof(float) + 8u * (((size_t)(hidden / 256u) * 210u + 15u) & ~(size_t)15u);
        const dim3 qgrid(grid.x + (with_shared ? 2u * ffn / 8u : 0u), ntok);
        REDHIP_LAUNCH(router_quant_kernel<T_Q6_K>, qgrid, dim3(256), lds, s, static_cast<const uint8_t *>(w), a);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------- softmax top-k selection by one wave

// Probabilities exactly as the CPU path forms them (expf(l - max), double sum, one float reciprocal). The wave
// holds all n_expert probabilities in registers (PER per lane, element i = lane + 64 * s). Non-negative floats
// order like their bit patterns, so the k-th largest probability is found by bisection on the bits with
// ballot/popcount; ties at the threshold are then taken in index order: exactly the set and order of an argmax
// loop with ties to the lower index. The k winners end up one per lane and are ranked against each other with
// lane broadcasts.
struct SelectOut {
    uint32_t ids[16];
    float w[16];
    float scalar;
    uint32_t tmp[64];
    float tmp_p[64];
    uint64_t cand[64];        // candidates: key << 32 | ~index
};


// (float)(1.0 / d) for finite d > 0 without the double division: a float reciprocal refined by two double FMAs is
// good to 2^-45, which rounds to the same float except in about one case in 2^20
__device__ __forceinline__ float reciprocal_as_float(double d) {
    const double r0 = (double)__builtin_amdgcn_rcpf((float)d);
    const double e = __builtin_fma(-d, r0, 1.0);
    return (float)__builtin_fma(r0, e, r0);
}

template <int PER>
__device__ __forceinline__ void wave_select_topk(const float *logits, uint32_t E, uint32_t K, SelectOut *out, float *probs = nullptr) {
    const uint32_t lane = threadIdx.x & 63u;
    float l[PER];
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < PER; ++s) {
        const uint32_t i = lane + 64u * s;
        l[s] = i < E ? logits[i] : -INFINITY;
        m = fmaxf(m, l[s]);
    }
    const float gate_logit = logits[E];                      // shared expert's gate logit rides along
    m = wave_max(m);
    REDHIP_STAMP(8);                                   // logits here, maximum known
    float p[PER];
    double part = 0.0;
#pragma unroll
    for (int s = 0; s < PER; ++s) {
        p[s] = lane + 64u * s < E ? expf(l[s] - m) : 0.0f;
        part += (double)p[s];
    }
    const double denom = wave_sum_d(part);
    const bool bad = !(denom > 0.0) || isinf(denom) || isnan(denom);
    const float inv = bad ? 0.0f : reciprocal_as_float(denom);
    REDHIP_STAMP(9);                                   // exponentials and their sum
    uint32_t key[PER];
#pragma unroll
    for (int s = 0; s < PER; ++s) {
        p[s] *= inv;
        key[s] = lane + 64u * s < E ? (__float_as_uint(p[s]) | 0x80000000u) : 0u;   // valid keys have the top bit set: padding never counts
        if (probs && lane + 64u * s < E) probs[lane + 64u * s] = p[s];
    }
    // Level 1: the K-th largest of the 64 per-lane maxima (tau) is a lower bound of the K-th largest key, so the
    // winners are among the keys >= tau - usually a dozen of them. Bisection on one value per lane is cheap.
    uint32_t lm = key[0];
#pragma unroll
    for (int s = 1; s < PER; ++s) lm = lm > key[s] ? lm : key[s];
    // Only the upper 16 bits of tau are searched (two per step): a smaller tau is still a lower bound, it only lets a
    // few more candidates through.
    uint32_t tau = 0x80000000u;                          // bit 31 is set in every valid key
#pragma unroll 1
    for (int bit = 29; bit >= 15; bit -= 2) {
        const uint32_t c1 = tau | (1u << bit), c2 = tau | (2u << bit), c3 = tau | (3u << bit);
        const uint32_t n1 = wave_count(lm >= c1), n2 = wave_count(lm >= c2), n3 = wave_count(lm >= c3);
        tau = n3 >= K ? c3 : n2 >= K ? c2 : n1 >= K ? c1 : tau;
    }
    uint32_t n_c = 0u;
#pragma unroll
    for (int s = 0; s < PER; ++s) n_c += wave_count(key[s] >= tau);
    REDHIP_STAMP(10);                                  // threshold and candidate count
    uint32_t mine = 0xffffffffu, kmine = 0u, rank = 0u;
    if (n_c <= 64u) {
        // Level 2: candidates to LDS in index order, one per lane, ranked against each other with lane broadcasts:
        // rank = number of candidates that beat this one under (p desc, index asc). rank < K <=> selected, and the
        // rank is the position in selection order.
        // A candidate is one 64-bit word, key above the complemented index: larger word <=> earlier in selection order.
        uint32_t n = 0u;
#pragma unroll
        for (int s = 0; s < PER; ++s) {
            const bool take = key[s] >= tau;
            const uint64_t mask = __ballot(take);
            if (take) {
                const uint32_t pos = n + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                out->cand[pos] = ((uint64_t)key[s] << 32) | (uint64_t)(~(lane + 64u * s));
            }
            n += (uint32_t)__popcll(mask);
        }
        if (lane >= n_c) out->cand[lane] = 0ull;                      // beats nobody
        wave_lds_sync();
        const uint64_t me = out->cand[lane];
        kmine = (uint32_t)(me >> 32);
        mine = lane < n_c ? ~(uint32_t)me : 0xffffffffu;
        // every lane reads the same entry (an LDS broadcast), 16 reads in flight at a time
        for (uint32_t base = 0; base < n_c; base += 16u) {
            uint64_t o[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) o[i] = out->cand[base + i];
#pragma unroll
            for (int i = 0; i < 16; ++i) rank += o[i] > me ? 1u : 0u;
        }
        if (lane >= n_c) { rank = 0xffffffffu; kmine = 0u; }
    } else {
        // Heavy ties (more than 64 keys at or above tau): bisection over all keys, ties at the threshold in index order.
        uint32_t T = 0x80000000u;
#pragma unroll 1
        for (int bit = 30; bit >= 0; --bit) {
            const uint32_t cand = T | (1u << bit);
            uint32_t c = 0u;
#pragma unroll
            for (int s = 0; s < PER; ++s) c += wave_count(key[s] >= cand);
            T = c >= K ? cand : T;
        }
        uint32_t above = 0u;
#pragma unroll
        for (int s = 0; s < PER; ++s) above += wave_count(key[s] > T);
        const uint32_t need_ties = K - above;                    // >= 1
        uint32_t n_sel = 0u, ties_seen = 0u;
#pragma unroll
        for (int s = 0; s < PER; ++s) {                          // index order = s-major over lanes
            const bool gt = key[s] > T, eq = key[s] == T;
            const uint64_t eq_mask = __ballot(eq);
            const uint32_t eq_before = ties_seen + (uint32_t)__popcll(eq_mask & ((1ull << lane) - 1ull));
            const bool take = gt || (eq && eq_before < need_ties);
            const uint64_t take_mask = __ballot(take);
            if (take) {
                const uint32_t pos = n_sel + (uint32_t)__popcll(take_mask & ((1ull << lane) - 1ull));
                out->tmp[pos] = lane + 64u * s;
                out->tmp_p[pos] = p[s];
            }
            n_sel += (uint32_t)__popcll(take_mask);
            ties_seen += (uint32_t)__popcll(eq_mask);
        }
        wave_lds_sync();
        if (lane < K) { mine = out->tmp[lane]; kmine = __float_as_uint(out->tmp_p[lane]) | 0x80000000u; }
        for (uint32_t q = 0; q < K; ++q) {
            const uint32_t o = __builtin_amdgcn_readlane(mine, q), ko = __builtin_amdgcn_readlane(kmine, q);
            rank += (ko > kmine || (ko == kmine && o < mine)) ? 1u : 0u;
        }
        if (lane >= K) rank = 0xffffffffu;
    }
    const bool selected = rank < K;
    REDHIP_STAMP(11);                                  // candidates ranked
    const float pm = __uint_as_float(kmine & 0x7fffffffu);
    const double sum = wave_sum_d(selected ? (double)pm : 0.0);
    const bool bad2 = bad || !(sum > 0.0) || isinf(sum) || isnan(sum);
    const float invs = bad2 ? __uint_as_float(0x7fc00000u) : reciprocal_as_float(sum);     // NaN weights flag an invalid softmax
    if (selected) {
        out->ids[rank] = mine < E ? mine : rank;
        out->w[rank] = pm * invs;
    }
    if (lane == 0u) out->scalar = 1.0f / (1.0f + expf(-gate_logit));
    REDHIP_STAMP(12);                                  // weights written
}

// ---------------------------------------------------------------- softmax top-k selection by a whole workgroup
//
// The same selection spread over the waves of a 1024-lane workgroup (one logit per lane in the first ceil(E / 64) waves), three
// barriers deep: a lone wave issues about one instruction per five clocks, so the single-wave routine above costs its instruction
// count; here every wave runs a short chain.
//   1. every selecting wave reads all logits for the maximum (same addresses in every wave, no barrier), then its own lane's
//      e = expf(l - max); per-wave double sums and the maxima of the 2 * NS half waves go to LDS.
//   2. denominator = the wave sums added in wave order; p = e * (float)(1 / denominator) as the CPU path forms it. The K-th largest
//      half-wave maximum (minus a few ulps: two different e can round to one p) bounds the K-th largest e from below, so the winners
//      are among the lanes at or above it, typically a dozen; each wave lists its candidates (p bits above the complemented index).
//   3. every candidate counts the candidates that beat it under (p descending, index ascending): that count is its place in selection
//      order, and the K lowest are the selected experts - the set and order of the CPU's argmax loop with ties to the lower index.
// Ties and degenerate inputs only lengthen the candidate lists (all-equal logits: every lane is a candidate), never change the result.
struct BlockSelect {
    double sum_part[16];
    uint32_t half_max[32];
    uint32_t cand_n[16];
    uint32_t ids[16];
    float p[16];
    uint64_t cand[16][64];      // per wave: its candidates in lane order; entries n .. kCandHead - 1 are zero (a zero beats nobody)
};
constexpr uint32_t kCandHead = 4u;      // candidates per wave that the ranking reads unconditionally (a wave rarely lists more)

__device__ __forceinline__ uint32_t umax32(uint32_t a, uint32_t b) { return a > b ? a : b; }
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u32(uint32_t v) { return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false); }
__device__ __forceinline__ uint32_t half_wave_max_u32(uint32_t v) {
    v = umax32(v, dpp_u32<kDppXor1>(v));
    v = umax32(v, dpp_u32<kDppXor2>(v));
    v = umax32(v, dpp_u32<kDppRor4>(v));
    v = umax32(v, dpp_u32<kDppRor8>(v));
    const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);      // rows 0 | 1 and rows 2 | 3 meet
    return umax32((uint32_t)r[0], (uint32_t)r[1]);
}

// Called by every thread of a workgroup of 16 waves; on return (behind a barrier) bs->ids[k], bs->p[k], k < K, hold the selection.
// NSM: upper bound of the waves that hold logits (8 for E <= 512, else 16). Every loop over waves is unrolled to it with predicates, so
// that the loads of one step (device memory for the logits, LDS afterwards) are all in flight together instead of one round trip each.
template <int NSM>
__device__ __forceinline__ void block_select_topk(const float *logits, uint32_t E, uint32_t K, BlockSelect *bs, float *probs = nullptr) {
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
    const uint32_t NS = (E + 63u) >> 6;                      // waves that hold logits (<= NSM)
    const bool valid = tid < E;
    float e = 0.0f;
    uint32_t ekey = 0u;
    if (wave < NS) {
        float lv[NSM];
#pragma unroll
        for (int s = 0; s < NSM; ++s) { const uint32_t q = lane + 64u * s; lv[s] = q < E ? logits[q] : -INFINITY; }
        const float l = valid ? logits[tid] : -INFINITY;
        float m = lv[0];
#pragma unroll
        for (int s = 1; s < NSM; ++s) m = fmaxf(m, lv[s]);
        m = wave_max(m);
        e = valid ? expf(l - m) : 0.0f;
        const double part = wave_sum_d((double)e);
        ekey = valid ? (__float_as_uint(e) | 0x80000000u) : 0u;      // valid keys have the top bit set: padding never counts
        const uint32_t hm = half_wave_max_u32(ekey);
        if (lane == 0u) bs->sum_part[wave] = part;
        if ((lane & 31u) == 0u) bs->half_max[2u * wave + (lane >> 5)] = hm;
    }
    __syncthreads();
    float p = 0.0f;
    uint64_t word = 0ull;
    bool take = false;
    if (wave < NS) {
        double sp[NSM];
#pragma unroll
        for (int w = 0; w < NSM; ++w) sp[w] = bs->sum_part[w];
        uint32_t hmx[2 * NSM];
#pragma unroll
        for (int q = 0; q < 2 * NSM; ++q) hmx[q] = bs->half_max[q];
        double denom = 0.0;
#pragma unroll
        for (int w = 0; w < NSM; ++w) denom += (uint32_t)w < NS ? sp[w] : 0.0;      // wave order
        const bool bad = !(denom > 0.0) || isinf(denom) || isnan(denom);
        p = e * (bad ? 0.0f : reciprocal_as_float(denom));
        const uint32_t key = valid ? (__float_as_uint(p) | 0x80000000u) : 0u;
        if (probs && valid) probs[tid] = p;
        const uint32_t NH = 2u * NS;
        uint32_t tau = 0x80000000u;                          // no bound: every valid lane is a candidate
        if (K <= NH) {
            const uint32_t v = lane < NH ? bs->half_max[lane] : 0u;
            uint32_t above = 0u;
#pragma unroll
            for (int q = 0; q < 2 * NSM; ++q) above += ((uint32_t)q < NH && (hmx[q] > v || (hmx[q] == v && (uint32_t)q < lane))) ? 1u : 0u;
            const uint64_t hit = __ballot(lane < NH && above == K - 1u);      // exactly one lane
            const uint32_t kth = (uint32_t)__shfl((int)v, __ffsll((long long)hit) - 1, 64);
            tau = kth > 0x80000004u ? kth - 4u : 0x80000000u;
        }
        take = valid && ekey >= tau;
        word = ((uint64_t)key << 32) | (uint64_t)(~tid);     // larger word <=> earlier in selection order
        const uint64_t mask = __ballot(take);
        const uint32_t n = (uint32_t)__popcll(mask);
        if (take) bs->cand[wave][__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u))] = word;
        if (lane >= n && lane < kCandHead) bs->cand[wave][lane] = 0ull;
        if (lane == 0u) bs->cand_n[wave] = n;
    }
    __syncthreads();
    if (wave < NS) {
        uint32_t rank = 0u;
#pragma unroll
        for (int w0 = 0; w0 < NSM; w0 += 8) {          // eight waves' lists at a time: 32 words in registers
            if ((uint32_t)w0 < NS) {
                uint64_t head[8][kCandHead];
                uint32_t cn[8];
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    cn[w] = bs->cand_n[w0 + w];
#pragma unroll
                    for (uint32_t q = 0; q < kCandHead; ++q) head[w][q] = bs->cand[w0 + w][q];
                }
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    if ((uint32_t)(w0 + w) < NS) {
#pragma unroll
                        for (uint32_t q = 0; q < kCandHead; ++q) rank += head[w][q] > word ? 1u : 0u;
                        const uint32_t n = (uint32_t)__builtin_amdgcn_readfirstlane((int)cn[w]);
                        for (uint32_t q = kCandHead; q < n; ++q) rank += bs->cand[w0 + w][q] > word ? 1u : 0u;      // a crowded wave: the rest of its list
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (take && rank < K) { bs->ids[rank] = tid; bs->p[rank] = p; }
    }
    __syncthreads();
}
// weight of selected expert k: p_k * (float)(1 / sum of the selected p in selection order, in double); NaN flags an invalid softmax
__device__ __forceinline__ float block_select_weight(const BlockSelect *bs, uint32_t K, uint32_t k) {
    float pp[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) pp[q] = bs->p[q];           // entries K .. 15 are never written: not added below
    double sum = 0.0;
#pragma unroll
    for (int q = 0; q < 16; ++q) sum += (uint32_t)q < K ? (double)pp[q] : 0.0;
    const bool bad = !(sum > 0.0) || isinf(sum) || isnan(sum);
    return bs->p[k] * (bad ? __uint_as_float(0x7fc00000u) : reciprocal_as_float(sum));
}

// stand-alone selection (one wave per token): ids / weights [ntok][top_k], scalar [ntok]
__global__ __launch_bounds__(64) void select_kernel(const float *logits, uint32_t E, uint32_t K, uint32_t *ids, float *weights, float *scalar,
                                                    float *probs) {
    __shared__ SelectOut sel;
    const float *l = logits + (uint64_t)blockIdx.x * (E + 1u);
    float *pr = probs ? probs + (uint64_t)blockIdx.x * E : nullptr;
    if (E <= 512u) wave_select_topk<8>(l, E, K, &sel, pr); else wave_select_topk<16>(l, E, K, &sel, pr);
    wave_lds_sync();
    if (threadIdx.x < K) {
        ids[(uint64_t)blockIdx.x * K + threadIdx.x] = sel.ids[threadIdx.x];
        weights[(uint64_t)blockIdx.x * K + threadIdx.x] = sel.w[threadIdx.x];
    }
    if (threadIdx.x == 0u && scalar) scalar[blockIdx.x] = sel.scalar;
}

// the same by a workgroup of 16 waves per token
__global__ __launch_bounds__(kWaves * 64) void select_block_kernel(const float *logits, uint32_t E, uint32_t K, uint32_t *ids, float *weights, float *scalar,
                                                                   float *probs) {
    __shared__ BlockSelect bs;
    const float *l = logits + (uint64_t)blockIdx.x * (E + 1u);
    float *pr = probs ? probs + (uint64_t)blockIdx.x * E : nullptr;
    if (E <= 512u) block_select_topk<8>(l, E, K, &bs, pr); else block_select_topk<16>(l, E, K, &bs, pr);
    if (threadIdx.x < K) {
        ids[(uint64_t)blockIdx.x * K + threadIdx.x] = bs.ids[threadIdx.x];
        weights[(uint64_t)blockIdx.x * K + threadIdx.x] = block_select_weight(&bs, K, threadIdx.x);
    }
    if (threadIdx.x == 0u && scalar) scalar[blockIdx.x] = 1.0f / (1.0f + expf(-l[E]));
}

hipError_t launch_select(const float *logits, uint32_t ntok, uint32_t n_expert, uint32_t top_k, uint32_t *ids, float *weights, float *scalar,
                         float *probs, hipStream_t s) {
    if (!ntok || !n_expert || n_expert > 1024u || !top_k || top_k > 16u || top_k > n_expert) return hipErrorInvalidValue;
    // few tokens: one workgroup of 16 waves each (short chains per wave); many tokens: one wave each (the machine is full either way)
    if (ntok <= 64u) REDHIP_LAUNCH(select_block_kernel, dim3(ntok), dim3(kWaves * 64), 0, s, logits, n_expert, top_k, ids, weights, scalar, probs);
    else REDHIP_LAUNCH(select_kernel, dim3(ntok), dim3(64), 0, s, logits, n_expert, top_k, ids, weights, scalar, probs);
    return hipGetLastError();
}

// Small batches routed by the layer's own router: wave t selects the experts of token t, then the whole workgroup sorts the pairs by
// expert (with the pass list of the batched expert-slice kernel). One workgroup; logits [ntok][n_expert + 1]; at most
// kSelectGroupTokens tokens and kGroupMaxPairs pairs.
constexpr uint32_t kSelectGroupTokens = 32u;
template <uint32_t TOK>      // tokens the workgroup has room for: 16 (a wave each) or kSelectGroupTokens
__global__ __launch_bounds__(kWaves * 64) void select_group_kernel(const float *logits, uint32_t ntok, uint32_t E, uint32_t K, uint32_t *ids, float *weights,
                                                                   float *scalar, GroupJob job) {
    __shared__ SelectOut sel[TOK];
    __shared__ uint32_t group_lds[kGroupLdsWords];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    for (uint32_t t = wave; t < ntok; t += (uint32_t)kWaves) {      // (more than sixteen tokens: a wave selects for two)
        const float *l = logits + (uint64_t)t * (E + 1u);
        if (E <= 512u) wave_select_topk<8>(l, E, K, &sel[t]); else wave_select_topk<16>(l, E, K, &sel[t]);
        wave_lds_sync();
        if (lane < K) { ids[t * K + lane] = sel[t].ids[lane]; weights[t * K + lane] = sel[t].w[lane]; }
        if (lane == 0u) scalar[t] = sel[t].scalar;
    }
    __syncthreads();
    group_small(job, group_lds, [&](uint32_t t, uint32_t k) { return sel[t].ids[k]; }, [&](uint32_t t, uint32_t k) { return sel[t].w[k]; });
}

hipError_t launch_select_group(const float *logits, uint32_t ntok, uint32_t n_expert, uint32_t top_k, uint32_t *ids, float *weights, float *scalar,
                               const GroupJob &job, hipStream_t s) {
    if (!ntok || ntok > kSelectGroupTokens || !n_expert || n_expert > 1024u || !top_k || top_k > 16u || top_k > n_expert || ntok * top_k > kGroupMaxPairs) return hipErrorInvalidValue;
    GroupJob gj = job;
    gj.ids = nullptr;
    gj.weights = nullptr;
    gj.ntok = ntok; gj.top_k = top_k; gj.n_expert = n_expert;
    if (ntok <= (uint32_t)kWaves) REDHIP_LAUNCH(select_group_kernel<kWaves>, dim3(1), dim3(kWaves * 64), 0, s, logits, ntok, n_expert, top_k, ids, weights, scalar, gj);
    else REDHIP_LAUNCH(select_group_kernel<kSelectGroupTokens>, dim3(1), dim3(kWaves * 64), 0, s, logits, ntok, n_expert, top_k, ids, weights, scalar, gj);
    return hipGetLastError();
}

// The pair sort of a caller's routing as a launch of its own, for batches beyond what the side job of another launch takes (17..32
// tokens, up to 512 pairs): one workgroup of 16 waves.
__global__ __launch_bounds__(kWaves * 64) void group_small_kernel(GroupJob job) {
    __shared__ uint32_t group_lds[kGroupLdsWords];
    group_small_given(job, group_lds);
}

hipError_t launch_group_small(const GroupJob &job, hipStream_t s) {
    if (!job.ids || !job.weights || !job.ntok || job.ntok > kSelectGroupTokens || !job.top_k || job.top_k > 16u || job.ntok * job.top_k > kGroupMaxPairs ||
        !job.n_expert || job.n_expert > 1024u) return hipErrorInvalidValue;
    REDHIP_LAUNCH(group_small_kernel, dim3(1), dim3(kWaves * 64), 0, s, job);
    return hipGetLastError();
}

// without a router (callers that bring their own routing): fp16 split of x and the scalar gate, one workgroup per token.
// NV > 0: hidden = 256 * NV and a thread keeps its NV activations in registers, so x is read once and the two block-wide
// reductions (largest |x|, gate_inp . x) share one barrier; NV == 0: any hidden, x read twice.
template <int NV>
__global__ __launch_bounds__(256) void prep_kernel(const float *x, const float *gate_inp, uint32_t H, _Float16 *xh, _Float16 *xl, int *xexp, float *scalar,
                                                   uint32_t ntok, GroupJob job) {
    __shared__ float red[8];
    __shared__ uint32_t group_lds[kGroupLdsWords];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u, tok = blockIdx.x;
    if (tok == ntok) {                                   // the extra workgroup: pair sort of the caller's routing
        group_small_given(job, group_lds);
        return;
    }
    const float *xt = x + (uint64_t)tok * H;
    float amax = 0.0f, acc = 0.0f;
    float xv[NV > 0 ? NV : 1];
    if constexpr (NV > 0) {
        float gv[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) { xv[k] = xt[threadIdx.x + 256u * k]; gv[k] = gate_inp[threadIdx.x + 256u * k]; }
#pragma unroll
        for (int k = 0; k < NV; ++k) { amax = fmaxf(amax, fabsf(xv[k])); acc = fmaf(gv[k], xv[k], acc); }
    } else {
        for (uint32_t i = threadIdx.x; i < H; i += 256u) { const float v = xt[i]; amax = fmaxf(amax, fabsf(v)); acc = fmaf(gate_inp[i], v, acc); }
    }
    amax = wave_max(amax);
    acc = wave_sum(acc);
    if (lane == 0u) { red[wave] = amax; red[4u + wave] = acc; }
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (threadIdx.x == 0u) scalar[tok] = 1.0f / (1.0f + expf(-((red[4] + red[5]) + (red[6] + red[7]))));
    const int e = prescale_exp(amax);
    const float inv = exp2i(-e);
    if constexpr (NV > 0) {
#pragma unroll
        for (int k = 0; k < NV; ++k) split_hi_lo(xv[k], inv, xh + (uint64_t)tok * H + threadIdx.x + 256u * k, xl + (uint64_t)tok * H + threadIdx.x + 256u * k);
    } else {
        for (uint32_t i = threadIdx.x; i < H; i += 256u) split_hi_lo(xt[i], inv, xh + (uint64_t)tok * H + i, xl + (uint64_t)tok * H + i);
    }
    if (threadIdx.x == 0u) xexp[tok] = e;
}

hipError_t launch_prep(const float *x, const float *gate_inp, uint32_t ntok, uint32_t hidden, void *xh, void *xl, int *xexp, float *scalar, hipStream_t s,
                       const GroupJob *job, bool *job_done) {
    const bool with_job = job && job_done && group_job_fits(*job);
    const dim3 grid(ntok + (with_job ? 1u : 0u));
    const GroupJob gj = with_job ? *job : GroupJob{};
    _Float16 *h = static_cast<_Float16 *>(xh), *l = static_cast<_Float16 *>(xl);
    switch (hidden) {
        case 512: REDHIP_LAUNCH(prep_kernel<2>, grid, dim3(256), 0, s, x, gate_inp, hidden, h, l, xexp, scalar, ntok, gj); break;
        case 1024: REDHIP_LAUNCH(prep_kernel<4>, grid, dim3(256), 0, s, x, gate_inp, hidden, h, l, xexp, scalar, ntok, gj); break;
        case 2048: REDHIP_LAUNCH(prep_kernel<8>, grid, dim3(256), 0, s, x, gate_inp, hidden, h, l, xexp, scalar, ntok, gj); break;
        case 4096: REDHIP_LAUNCH(prep_kernel<16>, grid, dim3(256), 0, s, x, gate_inp, hidden, h, l, xexp, scalar, ntok, gj); break;
        default: REDHIP_LAUNCH(prep_kernel<0>, grid, dim3(256), 0, s, x, gate_inp, hidden, h, l, xexp, scalar, ntok, gj); break;
    }
    if (job_done) *job_done = with_job;
    return hipGetLastError();
}

// ---------------------------------------------------------------- gate/up + SwiGLU and down + combine

template <int N, int OFF>
__device__ __forceinline__ void halve_step(float *v, uint32_t lane) {      // N live values -> N / 2
    const bool upper = (lane & (uint32_t)OFF) != 0u;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
        const float keep = upper ? v[N / 2 + i] : v[i];
        const float give = upper ? v[i] : v[N / 2 + i];
        v[i] = keep + __shfl_xor(give, OFF, 64);
    }
}
// sum of `v` over the 16 lanes that share lane % 4, for UPW values at once. A lane is (row = lane / 16, b = lane / 4 % 4,
// j = lane % 4). Swapping the upper 32 lanes of one value with the lower 32 of another and adding leaves each half of
// the wave with one value summed over both halves; the same with odd and even rows of 16 leaves row r with value r
// summed over all rows; two rotating adds inside the row finish the sum over b.
__device__ __forceinline__ float swap_add_32(float a, float b) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap_add_16(float a, float b) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float row_sum_b(float s) {
    s += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(s), 0x128, 0xf, 0xf, false));   // row_ror:8
    s += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(s), 0x124, 0xf, 0xf, false));   // row_ror:4
    return s;
}
template <int UPW>
__device__ __forceinline__ float quad_column_reduce(float *v, uint32_t lane) {
    static_assert(UPW == 1 || UPW == 2 || UPW == 4 || UPW == 8, "units per wave");
    if constexpr (UPW == 8) {
        halve_step<8, 32>(v, lane);
        halve_step<4, 16>(v, lane);
        halve_step<2, 8>(v, lane);
        return v[0] + __shfl_xor(v[0], 4, 64);
    } else if constexpr (UPW == 4) {
        return row_sum_b(swap_add_16(swap_add_32(v[0], v[2]), swap_add_32(v[1], v[3])));
    } else if constexpr (UPW == 2) {
        const float h = swap_add_32(v[0], v[1]);
        return row_sum_b(swap_add_16(h, h));
    } else {
        const float h = swap_add_32(v[0], v[0]);
        return row_sum_b(swap_add_16(h, h));
    }
}
// the unit whose total a lane holds after quad_column_reduce, and whether this lane is the one that stores it
template <int UPW> __device__ __forceinline__ uint32_t reduced_unit(uint32_t lane) {
    uint32_t u = 0u;
    if constexpr (UPW >= 2) u += (lane & 32u) ? UPW / 2 : 0;
    if constexpr (UPW >= 4) u += (lane & 16u) ? UPW / 4 : 0;
    if constexpr (UPW >= 8) u += (lane & 8u) ? UPW / 8 : 0;
    return u;
}
template <int UPW> __device__ __forceinline__ bool reduced_writer(uint32_t lane) {
    constexpr uint32_t kPlainBits = UPW >= 8 ? 4u : UPW >= 4 ? 12u : UPW >= 2 ? 28u : 60u;   // lane bits folded by plain steps
    return (lane & kPlainBits) == 0u;
}

// 32 weights of one group against the lane's activation operand: (hi . w + lo . w * 2^-11) * (2 * scale + 1).
// v_mfma_f32_4x4x4_16B_f16: lanes 4b..4b+3 form block b; lane j of a block supplies row j of A (the activation
// halves: j = 0 hi, j = 1 lo, others zero) and column j of B (its own four weights), and receives column j of
// A x B: acc[0] = hi . w, acc[1] = lo . w.
__device__ __forceinline__ float group_dot(uint2 q, const half4_t *ax, const uint8_t *lds) {
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t idx = (q.x >> (8u * l)) & 255u, s7 = (q.y >> (7u * l)) & 127u;
        WeightQuad b0, b1;
        signed_weights(lds, idx, s7, b0, b1);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l], b0.h, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l + 1u], b1.h, acc, 0, 0, 0);
    }
    return (acc[0] + acc[1] * 4.8828125e-4f) * (float)(2u * (q.y >> 28) + 1u);
}

// The same product for the packed IQ2_XS group (FMT 1: 9-bit indices into the caller's 512-entry codebook, one scale per 16 weights in
// `sc`) and the packed IQ1_M group (FMT 2: 11-bit indices into the caller's 2048-entry codebook of -1 / 0 / 1, plus or minus 1/8 per
// eight weights added as packed fp16, exact; 3-bit scales per 16 weights in q.y). `lds` is the fp16 copy of the codebook.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// va: the product with the token in rows 0, 1 (hi, lo) of the activation operand, vb: with the one in rows 2, 3 (if any)
template <int FMT>
__device__ __forceinline__ void group_dot_fmt2(uint2 q, uint32_t sc, const half4_t *ax, const uint8_t *lds, float &va, float &vb) {
    static_assert(FMT == 1 || FMT == 2, "codebook formats");
    {
        float4_t acc[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
        for (uint32_t l = 0; l < 4u; ++l) {
            WeightQuad b0, b1;
            if constexpr (FMT == 1) {
                const uint32_t w16 = ((l < 2u ? q.x : q.y) >> (16u * (l & 1u))) & 0xffffu;
                signed_weights(lds, w16 & 511u, w16 >> 9, b0, b1);
            } else {
                const uint32_t idx = ((q.x >> (8u * l)) & 255u) | (((q.y >> (4u * l)) & 7u) << 8);
                const uint4 m = *reinterpret_cast<const uint4 *>(lds + (idx << 4));
                const half2_t delta = __builtin_bit_cast(half2_t, 0x30003000u | (((q.y >> (4u * l + 3u)) & 1u) * 0x80008000u));
                b0.u[0] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.x) + delta);
                b0.u[1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.y) + delta);
                b1.u[0] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.z) + delta);
                b1.u[1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.w) + delta);
            }
            acc[l >> 1] = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l], b0.h, acc[l >> 1], 0, 0, 0);
            acc[l >> 1] = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l + 1u], b1.h, acc[l >> 1], 0, 0, 0);
        }
        const uint32_t s0 = FMT == 1 ? (sc & 15u) : ((q.y >> 16) & 7u), s1 = FMT == 1 ? (sc >> 4) : ((q.y >> 19) & 7u);
        const float f0 = (float)(2u * s0 + 1u), f1 = (float)(2u * s1 + 1u);
        va = (acc[0][0] + acc[0][1] * 4.8828125e-4f) * f0 + (acc[1][0] + acc[1][1] * 4.8828125e-4f) * f1;
        vb = (acc[0][2] + acc[0][3] * 4.8828125e-4f) * f0 + (acc[1][2] + acc[1][3] * 4.8828125e-4f) * f1;
    }
}
template <int FMT>
__device__ __forceinline__ float group_dot_fmt(uint2 q, uint32_t sc, const half4_t *ax, const uint8_t *lds) {
    if constexpr (FMT == 0) {
        return group_dot(q, ax, lds);
    } else {
        float va, vb;
        group_dot_fmt2<FMT>(q, sc, ax, lds, va, vb);
        return va;
    }
}

// the lane's activation operand: 32 values starting at src (fp16), lanes j = 0 / 1 carry hi / lo, others zero
__device__ __forceinline__ void load_act_operand(half4_t *ax, const _Float16 *hi, const _Float16 *lo, uint32_t j) {
    const _Float16 *src = j == 0u ? hi : lo;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        half4_t v = {(_Float16)0, (_Float16)0, (_Float16)0, (_Float16)0};
        if (j < 2u) v = *reinterpret_cast<const half4_t *>(src + 4 * s);
        ax[s] = v;
    }
}

struct GateUpArgs {
    const uint8_t *experts;    // packed experts of the layer, expert e at experts + e * stride
    uint64_t stride;
    const int8_t *grid;        // the caller's codebook of the routed experts' format (IQ2_XS, IQ1_M) or nullptr
    const uint8_t *shared;     // packed shared expert, or nullptr when it is not IQ2_XXS
    const uint8_t *shared_q6k; // then: its raw Q6_K rows, gate matrix then up matrix
    const float *x;            // [hidden] f32 activations (Q6_K shared expert only)
    const float *shared_gu;    // or, instead of the two above: gate . x and up . x of the shared expert, [2 * ffn], already computed
    const float *logits;       // [n_expert + 1] (selection happens here) or nullptr: ids come from `ids_in`
    const uint32_t *ids_in;    // [top_k] when logits == nullptr
    uint32_t *ids_out;         // [top_k]   written by workgroup (0, 0) when selecting
    float *weights_out;        // [top_k]
    float *scalar_out;         // [1]
    const _Float16 *xh, *xl;   // [hidden]
    const int *xexp;           // [1]
    _Float16 *act_h, *act_l;   // [top_k + 1][ffn]
    int *act_exp;              // [top_k + 1][ffn / 32]
    uint32_t hidden, ffn, n_expert, top_k;
    uint32_t *status;          // RouteGuard::status when ids_in is the caller's
};

// FMT: format of the routed (and a packed shared) expert's gate / up matrices: 0 IQ2_XXS, 1 IQ2_XS, 2 IQ1_M
template <int NKC, int FMT>        // K chunks of 512 columns in a gate/up row: hidden = 512 * NKC
__global__ __launch_bounds__(kWaves * 64) void gateup_select_kernel(const float *logits_first, uint32_t n_expert_first, uint32_t top_k_first, GateUpArgs a) {
    constexpr int NW = kWaves;
    constexpr int UPW = 16 * NKC / NW;                 // (row-quad, K-chunk) units per wave
    static_assert(UPW >= 1 && UPW * NW == 16 * NKC, "waves must tile the 16 row-quads x NKC chunks");
    __shared__ __attribute__((aligned(16))) uint8_t lds[FMT == 0 ? kMagBytes : FMT == 1 ? 512u * 16u : 2048u * 16u];
    __shared__ float part[NKC * 64];
    __shared__ SelectOut sel;

    const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    // The leading kernel arguments repeat a.logits, a.n_expert, a.top_k: they can reach a wave in registers at its start, so the selecting
    // wave's request for the logits leaves before the argument block has come from memory - and before anything else this wave does.
    if (blockIdx.y < top_k_first && logits_first && wave == 0u) {
        const float *lg = logits_first + (uint64_t)blockIdx.z * (n_expert_first + 1u);
        if (n_expert_first <= 512u) wave_select_topk<8>(lg, n_expert_first, top_k_first, &sel);
        else wave_select_topk<16>(lg, n_expert_first, top_k_first, &sel);
    }
    const uint32_t H = a.hidden, F = a.ffn, HG = H / 32u, HB = H / 256u;
    if (const uint32_t tok = blockIdx.z) {             // several tokens in one launch: every token is a layer of the grid with buffers of its own
        const uint64_t t = tok;
        if (a.x) a.x += t * H;
        if (a.shared_gu) a.shared_gu += t * 2u * F;
        if (a.logits) a.logits += t * (a.n_expert + 1u);
        if (a.ids_in) a.ids_in += t * a.top_k;
        a.ids_out += t * a.top_k;
        a.weights_out += t * a.top_k;
        a.scalar_out += t;
        a.xh += t * H;
        a.xl += t * H;
        a.xexp += t;
        a.act_h += t * (a.top_k + 1u) * F;
        a.act_l += t * (a.top_k + 1u) * F;
        a.act_exp += t * (a.top_k + 1u) * (F / 32u);
    }
    const uint32_t g = blockIdx.x;                     // FFN column group: act values [32 g, 32 g + 32)
    const uint32_t slot = blockIdx.y;
    const bool is_shared = slot >= a.top_k;
    const uint32_t tb = tid - 256u;                     // waves 4..7 build the table: wave 0 goes straight to the selection
    const uint64_t grid_entry = FMT == 0 && tb < 256u ? redhip_iq2xxs_grid[tb] : 0ull;

    // activation operand: independent of the routing, requested before the selection
    const uint32_t kc = wave % NKC, q0 = wave / NKC;
    const uint32_t G = 16u * kc + blk;                 // this lane's group inside the gate/up rows
    half4_t ax[8];
    load_act_operand(ax, a.xh + 32u * G, a.xl + 32u * G, j);
    if constexpr (FMT == 0) build_tables(lds, tb, grid_entry);
    else if (!is_shared) build_codebook_table<FMT>(lds, tid, a.grid);      // a shared expert beside these formats is never packed

    uint32_t expert = 0u;
    extern __shared__ __attribute__((aligned(16))) uint8_t raw_rows[];      // Q6_K shared expert only: the unit's 64 raw rows, then x
    if (is_shared) {
        if (!a.shared && !a.shared_gu) {
            // wave w copies its rows 4 w .. 4 w + 3 of the unit (0..31 gate, 32..63 up; contiguous in their matrix) and a
            // share of x into LDS with wide loads, requested before anything else happens in this workgroup
            const uint32_t row_bytes = HB * 210u;
            const uint8_t *src = a.shared_q6k + (wave < 8u ? 0u : (uint64_t)F * row_bytes) + (uint64_t)(32u * g + 4u * (wave & 7u)) * row_bytes;
            wave_stage(raw_rows + 4u * wave * row_bytes, src, 4u * row_bytes, lane);
            float *xs = reinterpret_cast<float *>(raw_rows + 64u * row_bytes), *xsum = xs + H + H / 32u;
            for (uint32_t i = tid; i < H; i += NW * 64u) xs[i + (i >> 5)] = a.x[i];
            if (tid < H / 16u) {                             // sums of 16 consecutive activations (the Q6_K offset term)
                const float4 *xp = reinterpret_cast<const float4 *>(a.x + 16u * tid);
                const float4 v0 = xp[0], v1 = xp[1], v2 = xp[2], v3 = xp[3];
                xsum[tid] = (((v0.x + v0.y) + (v0.z + v0.w)) + ((v1.x + v1.y) + (v1.z + v1.w))) + (((v2.x + v2.y) + (v2.z + v2.w)) + ((v3.x + v3.y) + (v3.z + v3.w)));
            }
        }
        __syncthreads();                                   // tables; the shared expert does not depend on the routing
    } else if (a.logits) {
        __syncthreads();                                   // the selection (wave 0, at the kernel's head) and the tables
        expert = sel.ids[slot];
        if (g == 0u && slot == 0u) {
            if (tid < a.top_k) { a.ids_out[tid] = sel.ids[tid]; a.weights_out[tid] = sel.w[tid]; }
            if (tid == 0u) a.scalar_out[0] = sel.scalar;
        }
    } else {
        expert = guarded_id(a.ids_in[slot], a.n_expert, a.status);
        __syncthreads();                               // tables
    }
    if (is_shared && !a.shared && a.shared_gu) {           // the router launch has already multiplied the shared expert's rows
        if (tid < 32u) {
            const float gsum = a.shared_gu[32u * g + tid], usum = a.shared_gu[F + 32u * g + tid];
            const float act = (gsum / (1.0f + expf(-gsum))) * usum;
            float amax = fabsf(act);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const int e = prescale_exp(amax);
            split_hi_lo(act, exp2i(-e), a.act_h + (uint64_t)slot * F + 32u * g + tid, a.act_l + (uint64_t)slot * F + 32u * g + tid);
            if (tid == 0u) a.act_exp[slot * (F / 32u) + g] = e;
        }
        return;
    }
    if (is_shared && !a.shared) {
        // Q6_K shared expert: plain decode and f32 FMAs; wave w takes rows 4 w .. 4 w + 3 of the unit (0..31 gate, 32..63 up),
        // the 16 lanes of a row take every 16th chunk of 32 columns and meet by row-wide adds
        const uint32_t urow = 4u * wave + (lane >> 4), row_bytes = HB * 210u;
        const float *xs = reinterpret_cast<const float *>(raw_rows + 64u * row_bytes), *xsum = xs + H + H / 32u;   // x, one float of padding per 32
        const uint8_t *rowp = raw_rows + urow * row_bytes;
        float acc = 0.0f;
        for (uint32_t c = lane & 15u; c < HG; c += 16u) {
            float xv[32];
#pragma unroll
            for (int i = 0; i < 32; ++i) xv[i] = xs[33u * c + i];
            acc += q6k_dot32(rowp, c, xv, xsum[2u * c], xsum[2u * c + 1u]);
        }
        acc += dpp_f32<kDppXor1>(acc);
        acc += dpp_f32<kDppXor2>(acc);
        acc += dpp_f32<kDppRor4>(acc);
        acc += dpp_f32<kDppRor8>(acc);
        if ((lane & 15u) < (uint32_t)NKC) part[(lane & 15u) * 64u + urow] = (lane & 15u) == 0u ? acc : 0.0f;
        __syncthreads();
        if (tid < 32u) {
            float gsum = 0.0f, usum = 0.0f;
#pragma unroll
            for (int c = 0; c < NKC; ++c) { gsum += part[c * 64 + tid]; usum += part[c * 64 + 32 + tid]; }
            const float act = (gsum / (1.0f + expf(-gsum))) * usum;
            float amax = fabsf(act);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const int e = prescale_exp(amax);
            split_hi_lo(act, exp2i(-e), a.act_h + (uint64_t)slot * F + 32u * g + tid, a.act_l + (uint64_t)slot * F + 32u * g + tid);
            if (tid == 0u) a.act_exp[slot * (F / 32u) + g] = e;
        }
        return;
    }
    const uint8_t *ex = is_shared ? a.shared : a.experts + (uint64_t)expert * a.stride;
    const uint64_t sc_off = (uint64_t)F * HG * 8u + (uint64_t)F * HB * 2u;       // IQ2_XS: the scale bytes follow the two other streams
    const uint64_t gate_bytes = sc_off + (FMT == 1 ? (uint64_t)F * HG : 0u);
    const uint2 *gate_qs = reinterpret_cast<const uint2 *>(ex);
    const uint16_t *gate_ds = reinterpret_cast<const uint16_t *>(ex + (uint64_t)F * HG * 8u);
    const uint2 *up_qs = reinterpret_cast<const uint2 *>(ex + gate_bytes);
    const uint16_t *up_ds = reinterpret_cast<const uint16_t *>(ex + gate_bytes + (uint64_t)F * HG * 8u);

    uint2 wq[UPW];
    uint32_t wd[UPW], wsc[UPW];
#pragma unroll
    for (int u = 0; u < UPW; ++u) {
        const uint32_t quad = q0 + (NW / NKC) * u;     // 0..7 gate, 8..15 up
        const uint32_t r = 32u * g + 4u * (quad & 7u) + j;
        const uint2 *qs = quad < 8u ? gate_qs : up_qs;
        const uint16_t *ds = quad < 8u ? gate_ds : up_ds;
        wq[u] = qs[(uint64_t)r * HG + G];
        wd[u] = ds[(uint64_t)r * HB + (G >> 3)];
        wsc[u] = FMT == 1 ? (uint32_t)(ex + (quad < 8u ? 0u : gate_bytes) + sc_off)[(uint64_t)r * HG + G] : 0u;
    }
    float v[UPW];
#pragma unroll
    for (int u = 0; u < UPW; ++u) v[u] = group_dot_fmt<FMT>(wq[u], wsc[u], ax, lds) * scale_to_f32(wd[u]);
    const float tot = quad_column_reduce<UPW>(v, lane);
    if (reduced_writer<UPW>(lane)) {
        const uint32_t quad = q0 + (NW / NKC) * reduced_unit<UPW>(lane);
        part[kc * 64u + 4u * quad + j] = tot;
    }
    __syncthreads();
    if (tid < 32u) {
        float gsum = 0.0f, usum = 0.0f;
#pragma unroll
        for (int c = 0; c < NKC; ++c) { gsum += part[c * 64 + tid]; usum += part[c * 64 + 32 + tid]; }
        const float xs = (FMT == 2 ? 1.0f : 0.125f) * exp2i(a.xexp[0]);      // d/8 (IQ1_M: d) and the pre-scale of x
        gsum *= xs;
        usum *= xs;
        const float act = (gsum / (1.0f + expf(-gsum))) * usum;
        float amax = fabsf(act);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        const int e = prescale_exp(amax);
        split_hi_lo(act, exp2i(-e), a.act_h + (uint64_t)slot * F + 32u * g + tid, a.act_l + (uint64_t)slot * F + 32u * g + tid);
        if (tid == 0u) a.act_exp[slot * (F / 32u) + g] = e;
    }
}

// ---- word-packed IQ3_S (see the section on IQ3_S down matrices below for the format): the decode shared by the kernels that read it
constexpr uint32_t kIq3TableBytes = 512u * 8u;
// Column-sliced copy of a word-packed matrix: group g of row r. Eight rows of one group side by side (128 bytes), then the next group of the
// same eight rows: the workgroups that take one group of many rows (expert slices) read whole 128-byte lines, those that take every
// group of eight rows (one-token down kernel) one contiguous block.
__device__ __forceinline__ uint64_t iq3s_sliced_index(uint32_t g, uint32_t r, uint32_t groups, uint32_t nrows) {
#ifdef IQ3_PLAIN_CM
    return (uint64_t)g * nrows + r;
#else
    (void)nrows;
    return ((uint64_t)(r >> 3) * groups + g) * 8u + (r & 7u);
#endif
}
// LDS table: the four bytes of every grid entry as fp16; built by the first 512 lanes of a workgroup
__device__ __forceinline__ uint32_t iq3s_quads_seed(uint32_t tid) { return tid < 512u ? redhip_iq3s_grid[tid] : 0u; }
__device__ __forceinline__ void build_iq3s_quads_from(uint8_t *lds, uint32_t tid, uint32_t e) {
    if (tid < 512u) {
        uint32_t w2[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const _Float16 lo = (_Float16)(float)((e >> (16 * i)) & 255u), hi = (_Float16)(float)((e >> (16 * i + 8)) & 255u);
            w2[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint2 *>(lds + (size_t)tid * 8u) = make_uint2(w2[0], w2[1]);
    }
}
__device__ __forceinline__ void build_iq3s_quads(uint8_t *lds, uint32_t tid) { build_iq3s_quads_from(lds, tid, iq3s_quads_seed(tid)); }

// 32 weights (one uint4 of words) against an activation operand that carries one token (rows 0, 1 = hi, lo) or two (rows 2, 3 the
// second): va = first token's product, vb = the second's; scale nibble applied, d is not.
__device__ __forceinline__ void iq3s_group_dot(uint4 q, const half4_t *ax, const uint8_t *lds, float &va, float &vb) {
    const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint2 ma = *reinterpret_cast<const uint2 *>(lds + ((w4[l] & 511u) << 3)), mb = *reinterpret_cast<const uint2 *>(lds + (((w4[l] >> 9) & 511u) << 3));
        const uint32_t s8s = ((w4[l] >> 18) & 255u) << 8;          // sign bit k of the eight at bit 8 + k, as place_signs takes them
        WeightQuad b0, b1;
        b0.u[0] = (__umul24(s8s, (1u << 7) | (1u << 22)) & 0x80008000u) | ma.x;
        b0.u[1] = (__umul24(s8s, (1u << 5) | (1u << 20)) & 0x80008000u) | ma.y;
        b1.u[0] = (__umul24(s8s, (1u << 3) | (1u << 18)) & 0x80008000u) | mb.x;
        b1.u[1] = (__umul24(s8s, (1u << 1) | (1u << 16)) & 0x80008000u) | mb.y;
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l], b0.h, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l + 1u], b1.h, acc, 0, 0, 0);
    }
    const float sc = (float)(2u * ((q.x >> 26) & 15u) + 1u);
    va = (acc[0] + acc[1] * 4.8828125e-4f) * sc;
    vb = (acc[2] + acc[3] * 4.8828125e-4f) * sc;
}

// ---------------------------------------------------------------- one token: expert slices
//
// (Described for all-IQ2_XXS layers; MIX = 1 / 2 / 3 reads the down slices of IQ3_S words or IQ2_XS / IQ1_M streams and takes the shared
// expert from dense f32 copies, SLOTS takes the experts from the slots of a pool - see SliceArgs.)
// One workgroup per (slot, 32 ffn columns): it selects (or takes the caller's routing), multiplies its 32 gate rows and 32 up rows
// of the slot's expert, applies SwiGLU, keeps the 32 activations in LDS and multiplies them straight away with the matching 32
// columns of the expert's down matrix - all `hidden` rows - weighted by the slot's router weight. Gate / up and down weights are
// requested together, right after the selection, so the launch waits for weights once, and the activations never leave the
// compute unit. What leaves it is one partial output vector per workgroup, partial[slot][column group][hidden]; slice_sum_kernel
// adds the (top_k + 1) * ffn / 32 partial vectors in a fixed order. The down matrices are read from a column-sliced copy
// (qs [ffn / 32][hidden] uint2, ds [ffn / 256][hidden] fp16) so that a workgroup's slice is contiguous.
//
// REP copies of every entry of the magnitude table sit side by side in LDS, lane l reads copy l % REP: with REP = 16 the sixteen
// lanes that the LDS serves together always hit sixteen different 16-byte bank groups, whatever entries they ask for.
struct SliceArgs {
    const uint8_t *experts;        // packed experts: gate | up streams (row-major), expert e at experts + e * stride
    uint64_t stride;
    const uint8_t *down_cm;        // column-sliced packed down matrices, expert e at down_cm + e * down_stride
    uint64_t down_stride;
    const uint8_t *shared;         // packed shared expert: gate | up
    const uint8_t *shared_down_cm;
    const float *logits;           // [n_expert + 1]: selection happens here; or nullptr: the caller's routing below
    const uint32_t *ids_in;        // [top_k]
    const float *weights_in;       // [top_k]
    const float *scalar_in;        // [1] sigmoid of the shared expert's gate logit
    uint32_t *ids_out;             // [top_k] written by workgroup (0, 0) when selecting
    float *weights_out;            // [top_k]
    float *scalar_out;             // [1]
    const _Float16 *xh, *xl;       // [hidden]
    const int *xexp;               // [1]
    float *partial;                // [top_k + 1][ffn / 32][hidden]
    uint32_t hidden, ffn, n_expert, top_k;
    uint32_t *status;              // RouteGuard::status when ids_in is the caller's
    // SLOTS variant: the experts of a pool of slots. slot_table[k] = address of slot k's raw bytes, its re-laid copy (packed gate | up,
    // column-sliced down) lies shadow_off behind it; x / x1 = f32 activations (experts from x_split on read x1), split to fp16 halves here
    const uint64_t *slot_table;
    uint64_t shadow_off;
    const float *x, *x1;
    uint32_t x_split;
    // MIX 1 (IQ2_XXS gate / up, IQ3_S down, dense shared expert): down_cm holds the column-sliced word-packed IQ3_S matrices; the shared
    // expert comes as its gate . x and up . x products [2 ffn] f32 (left by the router launch) and the dense f32 copy [hidden][ffn] of its
    // down matrix
    const float *shared_gu, *shared_dense;
    // MIX 2 / 3: `experts` holds the row-major IQ2_XS / IQ1_M streams of gate | up, down_cm the column-sliced streams of the down matrices,
    // grid the caller's codebook; the shared expert as for MIX 1
    const int8_t *grid;
};

// Two tables, REP copies of every 16-byte entry side by side (entry i, copy c at (i * REP + c) * 16), lane l reads copy l % REP: with
// REP = 16 the sixteen lanes that the LDS serves together always hit sixteen different 16-byte bank groups, whatever entries they ask for.
//   magnitudes: 256 entries, the eight fp16 magnitudes of a grid entry;
//   sign masks: 128 entries, for a 7-bit sign field (the eighth sign is its parity) the four words that flip the fp16 sign bits of the
//               eight weights (bit 15 / 31 of word i = sign of weight 2 i / 2 i + 1) - one read and four XORs in place of a dozen integer
//               operations per eight weights.
// Built by NB whole waves (NB = 8 or 16; `bw` = index of this wave among them, other waves pass bw >= NB and do nothing). Wave bw owns
// 256 / NB grid entries and 128 / NB sign fields: its first lanes make one entry each in a compact strip (`strip`: 4 KB + 2 KB), then the
// wave copies every entry to its REP slots with lane % 16 = copy and lane / 16 = entry (conflict-free writes too). Nothing but the
// wave's own strip entries is read: no workgroup barrier inside.
constexpr uint32_t kSignBytes = 128u * 16u;
// SREP: copies of the sign table (16, or 8 where LDS is short: lanes l and l + 8 then share a copy and sometimes collide)
// The grid entry a lane turns into its strip entry comes from device memory: table_seed requests it (a kernel whose routing arrives by
// a load of its own asks for the seed first, so that both round trips are one), build_tables_rep_from does the rest.
template <int NB>
__device__ __forceinline__ uint64_t table_seed(uint32_t bw, uint32_t lane) {
    constexpr uint32_t kOwn = 256u / NB;
    return (bw < (uint32_t)NB && lane < kOwn) ? redhip_iq2xxs_grid[bw * kOwn + lane] : 0ull;
}
template <int REP, int NB, int SREP = REP>
__device__ __forceinline__ void build_tables_rep_from(uint8_t *lds, uint8_t *strip, uint32_t bw, uint32_t lane, uint64_t grid_entry) {
    static_assert((REP == 16 || REP == 8) && (SREP == 16 || SREP == 8 || SREP == 0) && (NB == 8 || NB == 16), "replication layout");
    if (bw >= (uint32_t)NB) return;
    constexpr uint32_t kOwn = 256u / NB, kOwnS = 128u / NB;      // entries of this wave
    uint8_t *sign_lds = lds + REP * kMagBytes, *sign_strip = strip + kMagBytes;
    if (lane < kOwn) {
        const uint32_t idx = bw * kOwn + lane;
        uint32_t w4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const _Float16 lo = (_Float16)(float)((uint32_t)(grid_entry >> (16 * i)) & 255u), hi = (_Float16)(float)((uint32_t)(grid_entry >> (16 * i + 8)) & 255u);
            w4[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint4 *>(strip + (size_t)idx * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    } else if (SREP != 0 && lane - 32u < kOwnS) {        // (kOwn <= 32)
        const uint32_t s7 = bw * kOwnS + lane - 32u, s8 = s7 | ((__popc(s7) & 1u) << 7);
        uint32_t w4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w4[i] = (((s8 >> (2 * i)) & 1u) << 15) | (((s8 >> (2 * i + 1)) & 1u) << 31);
        *reinterpret_cast<uint4 *>(sign_strip + (size_t)s7 * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
    wave_lds_sync();
    constexpr uint32_t kPerM = 64u / REP;                // entries per copy instruction
#pragma unroll
    for (uint32_t k = 0; k < kOwn / kPerM; ++k) {
        const uint32_t idx = bw * kOwn + kPerM * k + lane / REP;
        const uint4 e = *reinterpret_cast<const uint4 *>(strip + (size_t)idx * 16u);
        *reinterpret_cast<uint4 *>(lds + ((size_t)idx * REP + lane % REP) * 16u) = e;
    }
    if constexpr (SREP != 0) {
        constexpr uint32_t kPer = 64u / (SREP ? SREP : 1);
#pragma unroll
        for (uint32_t k = 0; k < kOwnS / kPer; ++k) {
            const uint32_t s7 = bw * kOwnS + kPer * k + lane / (SREP ? SREP : 1);
            const uint4 e = *reinterpret_cast<const uint4 *>(sign_strip + (size_t)s7 * 16u);
            *reinterpret_cast<uint4 *>(sign_lds + ((size_t)s7 * SREP + lane % (SREP ? SREP : 1)) * 16u) = e;
        }
    }
}
template <int REP, int NB, int SREP = REP>
__device__ __forceinline__ void build_tables_rep(uint8_t *lds, uint8_t *strip, uint32_t bw, uint32_t lane) {
    build_tables_rep_from<REP, NB, SREP>(lds, strip, bw, lane, table_seed<NB>(bw, lane));
}
// eight signed fp16 weights from the two replicated tables; `tab` / `stab` = base of the magnitude / sign table + this lane's copy offset
template <int REP, int SREP>
__device__ __forceinline__ void signed_weights_rep(const uint8_t *tab, const uint8_t *stab, uint32_t idx, uint32_t s7, WeightQuad &b0, WeightQuad &b1) {
    const uint4 m = *reinterpret_cast<const uint4 *>(tab + idx * (16u * REP));
    const uint4 sg = *reinterpret_cast<const uint4 *>(stab + s7 * (16u * SREP));
    b0.u[0] = m.x ^ sg.x;
    b0.u[1] = m.y ^ sg.y;
    b1.u[0] = m.z ^ sg.z;
    b1.u[1] = m.w ^ sg.w;
}
// group_dot on the replicated tables
template <int REP, int SREP>
__device__ __forceinline__ float group_dot_rep(uint2 q, const half4_t *ax, const uint8_t *tab, const uint8_t *stab) {
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t idx = (q.x >> (8u * l)) & 255u, s7 = (q.y >> (7u * l)) & 127u;
        WeightQuad b0, b1;
        signed_weights_rep<REP, SREP>(tab, stab, idx, s7, b0, b1);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l], b0.h, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l + 1u], b1.h, acc, 0, 0, 0);
    }
    return (acc[0] + acc[1] * 4.8828125e-4f) * (float)(2u * (q.y >> 28) + 1u);
}

// Signs from a small table instead of a table of whole masks: entry s7 is ONE word that holds the eight sign bits of the field (the eighth
// = its parity) where shifts of 0..3 put them on the fp16 sign positions of the four weight pairs - bit 15 - i / 31 - i = sign of weight
// 2 i / 2 i + 1. A pair of signed weights is then (entry << i) & 0x80008000 | magnitudes: seven operations per eight weights and a 4-byte
// read, against a 16-byte read and four XORs for the table of masks, or thirteen operations without a table.
// LR copies of every entry side by side (entry s7, copy c at (s7 * LR + c) * 4), lane l reads copy l % LR.
__device__ __forceinline__ uint32_t spread_signs(uint32_t s7) {
    const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
    uint32_t e = 0u;
#pragma unroll
    for (uint32_t i = 0; i < 4u; ++i) e |= (((s8 >> (2u * i)) & 1u) << (15u - i)) | (((s8 >> (2u * i + 1u)) & 1u) << (31u - i));
    return e;
}
template <int LR>      // written by `builders` lanes starting at lane `first` of the workgroup (lanes before `first` wrap past the bound and write nothing)
__device__ __forceinline__ void build_sign_lut(uint32_t *lut, uint32_t tid, uint32_t first = 0u, uint32_t builders = (uint32_t)kWaves * 64u) {
    for (uint32_t n = tid - first; n < 128u * LR; n += builders) lut[n] = spread_signs(n / LR);
}
// The same words as data, for kernels that would rather request a word early than compute it (thirty operations per word)
struct SignWordTable { uint32_t w[128]; };
constexpr SignWordTable make_sign_words() {
    SignWordTable t{};
    for (uint32_t s7 = 0; s7 < 128u; ++s7) {
        uint32_t par = 0u;
        for (uint32_t b = 0; b < 7u; ++b) par ^= (s7 >> b) & 1u;
        const uint32_t s8 = s7 | (par << 7);
        uint32_t e = 0u;
        for (uint32_t i = 0; i < 4u; ++i) e |= (((s8 >> (2u * i)) & 1u) << (15u - i)) | (((s8 >> (2u * i + 1u)) & 1u) << (31u - i));
        t.w[s7] = e;
    }
    return t;
}
__device__ const SignWordTable redhip_sign_words = make_sign_words();
// Where the two tables lie for a lane, as 32-bit LDS addresses with the lane's copy offset added in. The copy offsets occupy the address
// bits below the entry index and the table bases the bits above it - magnitudes (64 KB-aligned): entry << 8 | (lane % 16) << 4; sign
// words (aligned to their size): field << (2 + log2 LR) | (lane % LR) << 2 - so that an address is one byte permute resp. a shift and an
// and-or of the packed group word, with no add.
struct LaneTables { uint32_t mag_lane, lut_lane; };
typedef uint32_t lds_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const lds_u32x4 *lds_u32x4_ptr;
typedef __attribute__((address_space(3))) const uint32_t *lds_u32_ptr;
__device__ __forceinline__ uint32_t lds_address(const void *p) { return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p; }
template <int REP, int LR>
__device__ __forceinline__ LaneTables lane_tables(const uint8_t *mag, const uint8_t *lut, uint32_t lane) {
    static_assert(REP == 16 && (LR == 8 || LR == 16 || LR == 32), "address bit layout");
    return LaneTables{lds_address(mag) + (lane % (uint32_t)REP) * 16u, lds_address(lut) + (lane % (uint32_t)LR) * 4u};
}
// eight signed weights: group word pair q, index / sign field L (0..3)
template <int REP, int LR, uint32_t L>
__device__ __forceinline__ void signed_weights_lut(const LaneTables &t, uint2 q, WeightQuad &b0, WeightQuad &b1) {
    constexpr uint32_t kLutShift = LR == 8 ? 5u : LR == 16 ? 6u : 7u;      // log2 of the bytes per sign field
    // bytes of the magnitude address: [low byte of the lane's base, index byte L of q.x, upper two bytes of the lane's base]
    const uint32_t mag_at = __builtin_amdgcn_perm(q.x, t.mag_lane, 0x03020000u | ((4u + L) << 8));
    const uint32_t field = 7u * L < kLutShift ? q.y << (kLutShift - 7u * L) : q.y >> (7u * L - kLutShift);
    const uint32_t lut_at = (field & (127u << kLutShift)) | t.lut_lane;
#ifdef REDHIP_ABLATE_NO_LDS      // measurement builds only (build.py --ablate): the table reads replaced by register moves, results wrong
    const lds_u32x4 m = {mag_at, lut_at, mag_at ^ 0x1234u, lut_at + 7u};
    const uint32_t e = lut_at ^ mag_at;
#else
    const lds_u32x4 m = *reinterpret_cast<lds_u32x4_ptr>((uintptr_t)mag_at);
    const uint32_t e = *reinterpret_cast<lds_u32_ptr>((uintptr_t)lut_at);
#endif
#ifdef REDHIP_ABLATE_NO_SIGN     // ... the sign placement left out
    b0.u[0] = m.x ^ e; b0.u[1] = m.y; b1.u[0] = m.z; b1.u[1] = m.w;
#else
    b0.u[0] = (e & 0x80008000u) | m.x;
    b0.u[1] = ((e << 1) & 0x80008000u) | m.y;
    b1.u[0] = ((e << 2) & 0x80008000u) | m.z;
    b1.u[1] = ((e << 3) & 0x80008000u) | m.w;
#endif
}
template <int REP, int LR, uint32_t L>
__device__ __forceinline__ float4_t group_step_lut(const LaneTables &t, uint2 q, const half4_t *ax, float4_t acc) {
    WeightQuad b0, b1;
    signed_weights_lut<REP, LR, L>(t, q, b0, b1);
#ifdef REDHIP_ABLATE_NO_MFMA     // ... the matrix instructions left out (the decoded weights stay live)
    asm volatile("" :: "v"(b0.u[0]), "v"(b0.u[1]), "v"(b1.u[0]), "v"(b1.u[1]));
    return acc;
#else
    acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * L], b0.h, acc, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * L + 1u], b1.h, acc, 0, 0, 0);
#endif
}
// group_dot / group_dot2 on the replicated magnitude table and the sign words
template <int REP, int LR>
__device__ __forceinline__ float4_t group_acc_lut(const LaneTables &t, uint2 q, const half4_t *ax) {
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    acc = group_step_lut<REP, LR, 0u>(t, q, ax, acc);
    acc = group_step_lut<REP, LR, 1u>(t, q, ax, acc);
    acc = group_step_lut<REP, LR, 2u>(t, q, ax, acc);
    return group_step_lut<REP, LR, 3u>(t, q, ax, acc);
}
template <int REP, int LR>
__device__ __forceinline__ float group_dot_lut(uint2 q, const half4_t *ax, const LaneTables &t) {
    const float4_t acc = group_acc_lut<REP, LR>(t, q, ax);
    return (acc[0] + acc[1] * 4.8828125e-4f) * (float)(2u * (q.y >> 28) + 1u);
}
template <int REP, int LR>
__device__ __forceinline__ void group_dot2_lut(uint2 q, const half4_t *ax, const LaneTables &t, float &va, float &vb) {
    const float4_t acc = group_acc_lut<REP, LR>(t, q, ax);
    const float sc = (float)(2u * (q.y >> 28) + 1u);
    va = (acc[0] + acc[1] * 4.8828125e-4f) * sc;
    vb = (acc[2] + acc[3] * 4.8828125e-4f) * sc;
}

constexpr int kSliceLut = 32;      // copies of the sign words in the one-token kernel: 16 KB, every lane of a half wave its own bank
// LDS bytes of the decode tables at the head of the one-token kernel's dynamic LDS
template <int REP, int MIX> constexpr uint32_t slice_table_bytes() {
    return MIX == 2 ? 512u * 16u : MIX == 3 ? 2048u * 16u : (uint32_t)(REP + 1) * kMagBytes + 128u * 4u * (uint32_t)kSliceLut;
}
constexpr uint32_t kSliceSharedParts = 4u;      // workgroups per 32 columns of a dense shared expert (mixed layouts)
template <int NKC, int REP, bool SLOTS = false, int MIX = 0>        // hidden = 512 * NKC; MIX as in batch_slice_kernel
__global__ __launch_bounds__(kWaves * 64) void expert_slice_kernel(const void *p0_first, uint32_t n_expert_first, uint32_t top_k_first, const void *p1_first,
                                                                   const void *p2_first, uint32_t u0_first, uint32_t hidden_first, uint32_t ffn_first, SliceArgs a) {
    constexpr int NW = kWaves;
    constexpr int UPW = 16 * NKC / NW;                 // (row-quad, K-chunk) units of gate / up per wave
    constexpr int DU = (8 * NKC + NW - 1) / NW;        // units of 64 down rows per wave
    static_assert(UPW >= 1 && UPW * NW == 16 * NKC, "waves must tile the 16 row-quads x NKC chunks");
    constexpr int FMT = MIX >= 2 ? MIX - 1 : 0;            // format of the routed matrices as group_dot_fmt2 numbers them
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];
    uint8_t *lds = dyn;                                                    // REP copies of the 4 KB magnitude table (MIX 2 / 3: the fp16 codebook, once)
    uint8_t *sign_lut = dyn + REP * kMagBytes;                             // kSliceLut copies of the 128 sign words (aligned to their size)
    uint8_t *strip = sign_lut + 128u * 4u * kSliceLut;                     // 4 KB: the magnitude table once, as its builders make it
    float *part = reinterpret_cast<float *>(dyn + slice_table_bytes<REP, MIX>());      // [NKC][64]
    _Float16 *act_hl = reinterpret_cast<_Float16 *>(part + NKC * 64);      // [2][32]: hi, lo halves of the 32 activations
    float *act_scale = reinterpret_cast<float *>(act_hl + 64);             // [4]
    SelectOut *sel = reinterpret_cast<SelectOut *>(act_scale + 4);
    [[maybe_unused]] uint8_t *iq3_tab = reinterpret_cast<uint8_t *>(sel + 1);      // MIX 1: 4 KB, the IQ3_S grid as fp16

    const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    // Mixed layouts: the shared expert's dense slice is kSliceSharedParts workgroups (a quarter of the output rows each: 16 x hidden bytes of f32
    // per row-quarter would otherwise be the longest-running workgroup); they come first in the grid, the routed slots behind them
    const uint32_t g = blockIdx.x, slot = MIX != 0 && !SLOTS ? (blockIdx.y < kSliceSharedParts ? top_k_first : blockIdx.y - kSliceSharedParts) : blockIdx.y;
    // The leading kernel arguments repeat what the first requests of the kernel need - a.logits, a.xh, a.xl (SLOTS: a.slot_table, a.x,
    // a.x1 and a.x_split), a.n_expert, a.top_k: leading scalar arguments can be handed to a wave in registers at its start, so these
    // requests do not wait for the argument block to come from memory.
    const float *logits_first = SLOTS ? nullptr : static_cast<const float *>(p0_first);
    const bool is_shared = slot >= top_k_first;
    const bool selecting = !SLOTS && !is_shared && logits_first;
    REDHIP_STAMP(0);
    // (hidden and ffn are leading arguments too, and the branch below tests the leading copy of a.logits: the selecting wave reaches the
    // barrier without having touched the argument block, whose fetch would otherwise sit between its selection and the barrier)
    const uint32_t H = hidden_first, F = ffn_first, HG = H / 32u, HB = H / 256u, FG = F / 32u;
    if constexpr (MIX != 0 && !SLOTS) {
        if (is_shared) {       // the shared expert's slice from dense f32 data: SwiGLU of the 32 columns, then their part of every output row
            if (tid < 32u) {
                const float *gu = a.shared_gu + 32u * g + tid;
                const float gv = gu[0], uv = gu[F];
                part[tid] = (gv / (1.0f + expf(-gv))) * uv;
            }
            const float gate = logits_first ? 1.0f / (1.0f + expf(-logits_first[n_expert_first])) : a.scalar_in[0];
            __syncthreads();
            // eight lanes per output row, each lane four of the 32 columns: a wave-wide load reads the 128-byte slices of eight rows whole
            const uint32_t sub = tid & 7u;
            const float4 av = *reinterpret_cast<const float4 *>(part + 4u * sub);
            constexpr uint32_t kRows = (uint32_t)NW * 8u;      // rows per round of the workgroup
            float *out = a.partial + ((uint64_t)slot * FG + g) * H;
            const uint32_t h_end = (blockIdx.y + 1u) * (H / kSliceSharedParts);      // (hidden is a multiple of 512)
            for (uint32_t h0 = blockIdx.y * (H / kSliceSharedParts) + (tid >> 3); h0 < h_end; h0 += 4u * kRows) {      // four rounds' loads in flight
                float4 w4[4];
#pragma unroll
                for (uint32_t i = 0; i < 4u; ++i) {
                    const uint32_t h = h0 + i * kRows;
                    w4[i] = *reinterpret_cast<const float4 *>(a.shared_dense + (uint64_t)(h < h_end ? h : h0) * F + 32u * g + 4u * sub);
                }
#pragma unroll
                for (uint32_t i = 0; i < 4u; ++i) {
                    const uint32_t h = h0 + i * kRows;
                    float acc = fmaf(w4[i].w, av.w, fmaf(w4[i].z, av.z, fmaf(w4[i].y, av.y, w4[i].x * av.x)));
#pragma unroll
                    for (int o = 1; o < 8; o <<= 1) acc += __shfl_xor(acc, o, 64);
                    if (h < h_end && sub == 0u) out[h] = acc * gate;
                }
            }
            return;
        }
    }

    // activation operand of the gate / up rows: independent of the routing, requested first
    const uint32_t kc = wave % NKC, q0 = wave / NKC;
    const uint32_t G = 16u * kc + blk;
    half4_t ax[8];
    float4 xf[SLOTS ? 8 : 1];                          // SLOTS: the lane's 32 activations as f32 (lanes j = 0, 1), split behind the barrier
    uint64_t slot_base = 0u;
    if constexpr (SLOTS) {
        slot_base = static_cast<const uint64_t *>(p0_first)[slot];
        const float *x_first = static_cast<const float *>(p1_first), *x1_first = static_cast<const float *>(p2_first);
        const float *xs = (x1_first && slot >= u0_first ? x1_first : x_first) + 32u * G;
        float amax = 0.0f;
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) {
            xf[s8] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (j < 2u) xf[s8] = *reinterpret_cast<const float4 *>(xs + 4 * s8);
        }
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) amax = fmaxf(fmaxf(amax, fmaxf(fabsf(xf[s8].x), fabsf(xf[s8].y))), fmaxf(fabsf(xf[s8].z), fabsf(xf[s8].w)));
        amax = wave_max(amax);                         // waves kc = 0 .. NKC - 1 cover the whole vector between them
        if (lane == 0u) reinterpret_cast<float *>(sel)[wave] = amax;
    } else {
        const _Float16 *xh_g = static_cast<const _Float16 *>(p1_first) + 32u * G, *xl_g = static_cast<const _Float16 *>(p2_first) + 32u * G;
        // The selecting wave asks for the logits before anything else and for its activations only behind the selection (requested together,
        // the logits were measured to arrive 0.5 us later: the wave then waits for all its loads); the barrier behind the selection
        // waits for LDS only, so those late activations do not hold the workgroup up.
        if (selecting && wave == 0u) {
            if (n_expert_first <= 512u) wave_select_topk<8>(logits_first, n_expert_first, top_k_first, sel);
            else wave_select_topk<16>(logits_first, n_expert_first, top_k_first, sel);
        }
        load_act_operand(ax, xh_g, xl_g, j);
    }
    [[maybe_unused]] uint32_t seed_q3 = 0u;
    if constexpr (MIX == 1) seed_q3 = iq3s_quads_seed(tid);
    // the table is first read behind the barrier that ends the selection: wave 0 selects, waves 8..15 build meanwhile
    // (and waves 1..7 write the sign words)
    [[maybe_unused]] LaneTables lt{};
    if constexpr (MIX >= 2) {                          // the codebook as fp16, by the waves that do not select
        if (selecting) build_codebook_table<FMT>(lds, tid, a.grid);
        else build_codebook_table<FMT>(lds, tid, a.grid, 0u, (uint32_t)NW * 64u);
    } else {
        if (selecting) { build_tables_rep<REP, 8, 0>(lds, strip, wave - 8u, lane); if (wave < 8u) build_sign_lut<kSliceLut>(reinterpret_cast<uint32_t *>(sign_lut), tid, 64u, 7u * 64u); }
        else { build_tables_rep<REP, 16, 0>(lds, strip, wave, lane); build_sign_lut<kSliceLut>(reinterpret_cast<uint32_t *>(sign_lut), tid); }
        lt = lane_tables<REP, kSliceLut>(lds, sign_lut, lane);
    }
    if constexpr (MIX == 1) build_iq3s_quads_from(iq3_tab, tid, seed_q3);

    uint32_t expert = 0u;
    float comb;                                        // the slot's weight in the layer's output
    int x_exp = 0;
    if constexpr (SLOTS) {
        comb = a.weights_in[slot];
        __syncthreads();                               // table, the waves' largest |x|
        float amax = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) amax = fmaxf(amax, reinterpret_cast<const float *>(sel)[w]);
        x_exp = prescale_exp(amax);
        const float inv = exp2i(-x_exp);
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) {
            const float t[4] = {xf[s8].x * inv, xf[s8].y * inv, xf[s8].z * inv, xf[s8].w * inv};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const _Float16 h = (_Float16)t[c];
                ax[s8][c] = j == 0u ? h : (_Float16)((t[c] - (float)h) * 2048.0f);      // (lanes j >= 2 hold zeros: both halves are zero)
            }
        }
    } else if (is_shared) {
        comb = logits_first ? 1.0f / (1.0f + expf(-logits_first[n_expert_first])) : a.scalar_in[0];
        __syncthreads();                               // table
    } else if (logits_first) {
        lds_barrier();                                 // selection (by wave 0, at the kernel's head) and table: both in LDS
        expert = __builtin_amdgcn_readfirstlane(sel->ids[slot]);      // the same in every lane: the weights' base addresses stay scalar
        comb = sel->w[slot];
        if (g == 0u && slot == 0u) {
            if (tid < a.top_k) { a.ids_out[tid] = sel->ids[tid]; a.weights_out[tid] = sel->w[tid]; }
            if (tid == 0u) a.scalar_out[0] = sel->scalar;
        }
    } else {
        expert = __builtin_amdgcn_readfirstlane(guarded_id(a.ids_in[slot], a.n_expert, a.status));
        comb = a.weights_in[slot];
        __syncthreads();                               // table
    }
    REDHIP_STAMP(1);                                   // selection (or the caller's routing) and tables are here
    const uint64_t gate_sc = (uint64_t)F * HG * 8u + (uint64_t)F * HB * 2u;       // IQ2_XS: the scale bytes [row][group] behind qs and ds
    const uint64_t gate_bytes = gate_sc + (MIX == 2 ? (uint64_t)F * HG : 0u);
    const uint8_t *ex = is_shared ? a.shared : a.experts + (uint64_t)expert * a.stride;
    const uint8_t *dn = is_shared ? a.shared_down_cm : a.down_cm + (uint64_t)expert * a.down_stride;
    if constexpr (SLOTS) {
        // (the builtin returns a signed int: each half goes through uint32_t, or a low half with bit 31 set would sign-extend over the high one)
        const uint32_t base_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)slot_base), base_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(slot_base >> 32));
        const uint64_t base = ((uint64_t)base_hi << 32) | base_lo;
        ex = reinterpret_cast<const uint8_t *>(base + a.shadow_off);
        dn = ex + 2u * gate_bytes;
    }
    // (bases the same in every lane, 32-bit byte offsets per lane: a matrix is far below 4 GB)
    using DownGroup = typename std::conditional<MIX == 1, uint4, uint2>::type;      // one row's 32 weights of the slice (IQ3_S: four words)
    const uint8_t *down_qs = dn + (MIX == 1 ? 0u : (uint64_t)g * H * 8u);                        // [FG][H] uint2; IQ3_S: blocks of eight rows per group
    const uint8_t *down_ds = dn + (uint64_t)FG * H * sizeof(DownGroup) + (uint64_t)(g >> 3) * H * 2u;      // [F / 256][H] fp16
    [[maybe_unused]] const uint8_t *down_sc = dn + ((uint64_t)FG * H * 8u + (uint64_t)(FG >> 3) * H * 2u + (uint64_t)g * H);      // MIX 2: [FG][H] scale bytes

    // every weight this workgroup needs is requested here: gate / up units, then the down slice
    uint2 wq[UPW];
    uint32_t wd[UPW];                                  // block scale d (fp16 bits); IQ2_XS: the group's scale byte above it
#pragma unroll
    for (int u = 0; u < UPW; ++u) {
        const uint32_t quad = q0 + (NW / NKC) * u;     // 0..7 gate, 8..15 up (the same in every lane of the wave)
        const uint32_t r = 32u * g + 4u * (quad & 7u) + j;
        const uint8_t *mat = ex + (quad < 8u ? 0u : gate_bytes);
        wq[u] = *reinterpret_cast<const uint2 *>(mat + (r * HG + G) * 8u);
        wd[u] = *reinterpret_cast<const uint16_t *>(mat + (F * HG * 8u + (r * HB + (G >> 3)) * 2u));
        if constexpr (MIX == 2) wd[u] |= (uint32_t)mat[(uint32_t)gate_sc + r * HG + G] << 16;
    }
    DownGroup dq[DU];
    uint32_t dd[DU];
#pragma unroll
    for (int k = 0; k < DU; ++k) {
        const uint32_t unit = wave + NW * k;           // 64 output rows each
        const uint32_t row = 64u * (unit < 8u * NKC ? unit : 0u) + lane;
        dq[k] = *reinterpret_cast<const DownGroup *>(down_qs + (MIX == 1 ? (uint32_t)iq3s_sliced_index(g, row, FG, H) : row) * (uint32_t)sizeof(DownGroup));
        dd[k] = *reinterpret_cast<const uint16_t *>(down_ds + row * 2u);
        if constexpr (MIX == 2) dd[k] |= (uint32_t)down_sc[row] << 16;
    }
    float v[UPW];
    REDHIP_STAMP(2);                                   // every weight requested
#pragma unroll
    for (int u = 0; u < UPW; ++u) {
        if constexpr (MIX >= 2) { float other; group_dot_fmt2<FMT>(wq[u], wd[u] >> 16, ax, lds, v[u], other); v[u] *= scale_to_f32(wd[u]); }
        else v[u] = group_dot_lut<REP, kSliceLut>(wq[u], ax, lt) * scale_to_f32(wd[u]);
        if (u == 0) REDHIP_STAMP(3);                   // the first unit's weights arrived and are multiplied
    }
    const float tot = quad_column_reduce<UPW>(v, lane);
    REDHIP_STAMP(4);                                   // gate / up rows of wave 0 multiplied
    if (reduced_writer<UPW>(lane)) {
        const uint32_t quad = q0 + (NW / NKC) * reduced_unit<UPW>(lane);
        part[kc * 64u + 4u * quad + j] = tot;
    }
    __syncthreads();
    REDHIP_STAMP(5);                                   // ... of every wave
    if (tid < 32u) {
        float gsum = 0.0f, usum = 0.0f;
#pragma unroll
        for (int c = 0; c < NKC; ++c) { gsum += part[c * 64 + tid]; usum += part[c * 64 + 32 + tid]; }
        const float xs = (MIX == 3 ? 1.0f : 0.125f) * exp2i(SLOTS ? x_exp : a.xexp[0]);      // d / 8 (an IQ1_M weight is d (2 s + 1) (entry +- 1/8): none) and the pre-scale of x
        gsum *= xs;
        usum *= xs;
        const float act = (gsum / (1.0f + expf(-gsum))) * usum;
        float amax = fabsf(act);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        const int e = prescale_exp(amax);
        split_hi_lo(act, exp2i(-e), act_hl + tid, act_hl + 32u + tid);
        if (tid == 0u) act_scale[0] = exp2i(e);
    }
    __syncthreads();
    REDHIP_STAMP(6);                                   // activations exchanged
    // down slice: lane = output row of the unit, the 32 activations are the same operand for every lane block
    half4_t ad[8];
    {
        const _Float16 *src = act_hl + (j == 1u ? 32u : 0u);
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) {
            half4_t t = {(_Float16)0, (_Float16)0, (_Float16)0, (_Float16)0};
            if (j < 2u) t = *reinterpret_cast<const half4_t *>(src + 4 * s8);
            ad[s8] = t;
        }
    }
    const float post = act_scale[0] * comb * (MIX == 1 || MIX == 3 ? 1.0f : 0.125f);     // the activations' pre-scale, the slot's weight, d / 8 (an IQ3_S weight is d (1 + 2 nibble) grid byte: no 1 / 8)
    float *out = a.partial + ((uint64_t)slot * FG + g) * H;
#pragma unroll
    for (int k = 0; k < DU; ++k) {
        const uint32_t unit = wave + NW * k;
        if (unit < 8u * NKC) {
            float dot;
            [[maybe_unused]] float other;
            if constexpr (MIX == 1) iq3s_group_dot(dq[k], ad, iq3_tab, dot, other);
            else if constexpr (MIX >= 2) group_dot_fmt2<FMT>(dq[k], dd[k] >> 16, ad, lds, dot, other);
            else dot = group_dot_lut<REP, kSliceLut>(dq[k], ad, lt);
            out[64u * unit + lane] = dot * scale_to_f32(dd[k]) * post;
        }
    }
    REDHIP_STAMP(7);                                   // down slice of wave 0 multiplied, stores issued
}

// out[r] = sum over slots (selection order, the shared expert last) and column groups of partial[slot][group][r] (+ the residual of the
// block step). 32 rows per workgroup as eight float4 columns; a thread adds every 32nd partial vector, the 32 threads of a column
// meet by shuffles and through LDS in a fixed order.
struct SumTail { const float *resid, *shared, *scalar; float *out2; };      // out = out2 = resid + (sum + shared * scalar[0]); all nullptr: none
__global__ __launch_bounds__(256) void slice_sum_kernel(const float *partial, uint32_t n_part, uint32_t H, float *out, const float *resid_a, const float *resid_b,
                                                        SumTail tail) {
    __shared__ float4 red[4][8];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u, c8 = tid & 7u, pl = tid >> 3;      // pl 0..31
    const uint32_t col = blockIdx.x * 8u + c8;          // float4 column
    const uint32_t H4 = H / 4u;
    const float4 *p4 = reinterpret_cast<const float4 *>(partial) + (uint64_t)blockIdx.y * n_part * H4;      // blockIdx.y = token
    out += (uint64_t)blockIdx.y * H;
    if (resid_a) { resid_a += (uint64_t)blockIdx.y * H; resid_b += (uint64_t)blockIdx.y * H; }
    float4 v[8];
    uint32_t n = 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t pp = pl + 32u * i;
        v[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (pp < n_part) { v[i] = p4[(uint64_t)pp * H4 + col]; n = i + 1; }
    }
    float4 acc = v[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) { acc.x += v[i].x; acc.y += v[i].y; acc.z += v[i].z; acc.w += v[i].w; }
    for (uint32_t base = 256u; base < n_part; base += 256u) {      // more than 256 partial vectors (large top_k x ffn)
        for (uint32_t pp = base + pl; pp < n_part && pp < base + 256u; pp += 32u) {
            const float4 t = p4[(uint64_t)pp * H4 + col];
            acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
        }
    }
    (void)n;
#pragma unroll
    for (int o = 8; o < 64; o <<= 1) {                  // lanes of a wave that share c8: lane bits 3..5
        acc.x += __shfl_xor(acc.x, o, 64); acc.y += __shfl_xor(acc.y, o, 64); acc.z += __shfl_xor(acc.z, o, 64); acc.w += __shfl_xor(acc.w, o, 64);
    }
    if (lane < 8u) red[wave][lane] = acc;
    __syncthreads();
    if (tid < 8u) {
        const float4 a0 = red[0][tid], a1 = red[1][tid], a2 = red[2][tid], a3 = red[3][tid];
        float4 sum = make_float4((a0.x + a1.x) + (a2.x + a3.x), (a0.y + a1.y) + (a2.y + a3.y), (a0.z + a1.z) + (a2.z + a3.z), (a0.w + a1.w) + (a2.w + a3.w));
        if (resid_a) {
            const float4 ra = reinterpret_cast<const float4 *>(resid_a)[col], rb = reinterpret_cast<const float4 *>(resid_b)[col];
            sum = make_float4((ra.x + rb.x) + sum.x, (ra.y + rb.y) + sum.y, (ra.z + rb.z) + sum.z, (ra.w + rb.w) + sum.w);
        }
        if (tail.resid) {
            const float4 r = reinterpret_cast<const float4 *>(tail.resid)[col], sh = reinterpret_cast<const float4 *>(tail.shared)[col];
            const float sc = tail.scalar[0];
            sum = make_float4(r.x + fmaf(sh.x, sc, sum.x), r.y + fmaf(sh.y, sc, sum.y), r.z + fmaf(sh.z, sc, sum.z), r.w + fmaf(sh.w, sc, sum.w));
            reinterpret_cast<float4 *>(tail.out2)[col] = sum;
        }
        reinterpret_cast<float4 *>(out)[col] = sum;
    }
}

// ---------------------------------------------------------------- two to eight tokens on all-IQ2_XXS layers: expert slices per pass
//
// The same slices for a small batch whose pairs are grouped by expert. A pass = up to two pairs (tokens) of one expert; one workgroup
// per (pass, 32 ffn columns): the two tokens ride in rows 0, 1 and 2, 3 of the MFMA's activation operand, so every weight is decoded
// once for both. A popular expert's tokens spread over several workgroups (its weights come from L2 after the first), the shared
// expert is one pass per two tokens. Partial vectors land at partial[token][k][column group][hidden] (k = top_k: the shared expert), so
// that the sum kernel reads one contiguous block per token.
struct BatchSliceArgs {
    const uint8_t *experts;
    uint64_t stride;
    const uint8_t *down_cm;
    uint64_t down_stride;
    const uint8_t *shared;
    const uint8_t *shared_down_cm;
    const uint2 *pass_list;        // from the pair sort (GroupJob::pass_list)
    const uint32_t *n_pass;
    const float *weights;          // [ntok][top_k] router weights, indexed token * top_k + k
    const float *scalar;           // [ntok]
    const _Float16 *xh, *xl;       // [ntok][hidden]
    const int *xexp;               // [ntok]
    float *partial;                // [ntok][top_k + 1][ffn / 32][hidden]
    uint32_t hidden, ffn, top_k, ntok;
    // mixed layouts (MIX): down_cm holds column-sliced word-packed IQ3_S matrices; the shared expert comes as its gate . x and up . x
    // products [ntok][2 ffn] f32 (left by the router launch) and the dense f32 copy [hidden][ffn] of its down matrix
    const float *shared_gu, *shared_dense;
    // MIX 2 / 3: `experts` holds the row-major IQ2_XS / IQ1_M streams of gate | up, down_cm the column-sliced streams of the down matrices,
    // grid the caller's codebook; the shared expert as for MIX 1
    const int8_t *grid;
};

// two tokens' results of one group: va for the token in rows 0, 1 of the operand, vb for the one in rows 2, 3
template <int REP, int SREP>
__device__ __forceinline__ void group_dot2_rep(uint2 q, const half4_t *ax, const uint8_t *tab, const uint8_t *stab, float &va, float &vb) {
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t idx = (q.x >> (8u * l)) & 255u, s7 = (q.y >> (7u * l)) & 127u;
        WeightQuad b0, b1;
        if constexpr (SREP == 0) place_signs(*reinterpret_cast<const uint4 *>(tab + idx * (16u * REP)), s7, b0, b1);
        else signed_weights_rep<REP, SREP>(tab, stab, idx, s7, b0, b1);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l], b0.h, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[2u * l + 1u], b1.h, acc, 0, 0, 0);
    }
    const float sc = (float)(2u * (q.y >> 28) + 1u);
    va = (acc[0] + acc[1] * 4.8828125e-4f) * sc;
    vb = (acc[2] + acc[3] * 4.8828125e-4f) * sc;
}

// One workgroup per (pass, column group) - the hardware's own dispatch balances the units over the compute units (persistent workgroups
// that walked a unit list with the next unit's weights requested ahead were measured too: slower at 2, 4 and 8 tokens, their start-up
// and the coarser balance cost more than the requests they hide).
// The magnitude table sixteen times, the signs placed by integer arithmetic (no sign table): 74 KB of LDS and at most 64 registers per
// lane, so that two workgroups fit a compute unit and one's weight requests and barriers hide behind the other's arithmetic. Measured
// at 8 tokens with 32 hot experts: this 27.7 us; eight copies of the magnitude table 28.3 us (38 % of its LDS cycles are bank
// conflicts: the LDS serves sixteen lanes of a 16-byte read together); eight copies of both tables 34.3 us (a fifth fewer vector
// instructions, 70 % more LDS reads); sixteen copies of both at one workgroup per compute unit 43.5 us.
constexpr int kBatchRep = 16, kBatchSignRep = 0, kBatchLut = 8;      // (kBatchLut copies of the 128 sign words: 4 KB)
// LDS bytes of the decode tables at the head of the kernel's dynamic LDS
template <int REP, int MIX> constexpr uint32_t batch_slice_table_bytes() {
    return MIX == 2 ? 512u * 16u : MIX == 3 ? 2048u * 16u : (uint32_t)(REP + 1) * kMagBytes + (uint32_t)kBatchSignRep * kSignBytes + 128u * 4u * (uint32_t)kBatchLut;
}
// MIX 0: every matrix packed IQ2_XXS; 1: IQ3_S down matrices, dense shared expert; 2 / 3: IQ2_XS / IQ1_M streams, dense shared expert (see BatchSliceArgs)
template <int NKC, int REP, int MIX>
__global__ __launch_bounds__(kWaves * 64, 8) void batch_slice_kernel(const uint2 *pass_list_first, const uint32_t *n_pass_first, uint32_t ntok_first, uint32_t top_k_first,
                                                                     BatchSliceArgs a) {
    constexpr int NW = kWaves;
    constexpr int UPW = 16 * NKC / NW;
    constexpr int DU = (8 * NKC + NW - 1) / NW;
    constexpr int SREP = kBatchSignRep;
    constexpr int FMT = MIX >= 2 ? MIX - 1 : 0;            // format of the routed matrices as group_dot_fmt2 numbers them
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];
    uint8_t *lds = dyn;
    uint8_t *strip = dyn + REP * kMagBytes + SREP * kSignBytes;            // 4 KB: the magnitude table once, as its builders make it
    uint8_t *sign_lut = strip + kMagBytes;                                 // kBatchLut copies of the sign words
    float *part = reinterpret_cast<float *>(dyn + batch_slice_table_bytes<REP, MIX>());      // [2 tokens][NKC][64]
    _Float16 *act_hl = reinterpret_cast<_Float16 *>(part + 2 * NKC * 64);  // [2 tokens][2 halves][32]
    float *act_scale = reinterpret_cast<float *>(act_hl + 128);            // [2] (+ 2 unused)
    uint8_t *iq3_tab = reinterpret_cast<uint8_t *>(act_scale + 4);         // MIX: 4 KB, the IQ3_S grid as fp16

    const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u, blk = lane >> 2, j = lane & 3u;      // (wave: in a scalar register)
    const uint32_t g = blockIdx.x, v = blockIdx.y, K = top_k_first;
    REDHIP_STAMP(0);
    // Three requests leave together, so that the workgroup waits for one round trip before it knows its weights' addresses: the number of
    // passes, this workgroup's entry of the pass list (read whether or not it turns out to be one: the index is clamped into the list) and
    // the codebook entries its lanes turn into the LDS tables. The tables are then written while the weights are on their way: loads
    // return in order, so a table seed requested behind the weights would not be usable before they have all arrived.
    // (the four leading kernel arguments repeat a.pass_list, a.n_pass, ntok_first, top_k_first: they can reach the wave in registers at its start,
    // so these requests do not wait for the argument block to come from memory)
    const uint32_t n_pairs = ntok_first * K;
    const uint32_t n_pass = n_pass_first[0];
    uint2 e = pass_list_first[v < n_pairs ? v : n_pairs - 1u];
    const uint32_t H = a.hidden, F = a.ffn, HG = H / 32u, HB = H / 256u, FG = F / 32u;
    uint64_t seed_cb[2] = {0ull, 0ull};
    uint64_t seed_mag = 0ull;
    uint32_t seed_q3 = 0u;
    uint32_t seed_sign = 0u;                           // kBatchLut = 8 copies of 128 words: one word per lane of the workgroup
    static_assert(kBatchLut * 128 == kWaves * 64, "one sign word per lane");
    if constexpr (MIX >= 2) codebook_seed<FMT>(tid, a.grid, seed_cb);
    else { seed_mag = table_seed<16>(wave, lane); seed_sign = redhip_sign_words.w[tid / (uint32_t)kBatchLut]; }
    if constexpr (MIX == 1) seed_q3 = iq3s_quads_seed(tid);
    if (v >= n_pass + ((ntok_first + 1u) >> 1)) return;    // the grid covers the largest possible number of passes
    const bool sh = v >= n_pass;
    if (sh) {                                          // the shared expert: tokens 2 s, 2 s + 1; k = top_k
        const uint32_t t0 = 2u * (v - n_pass), t1 = t0 + 1u < ntok_first ? t0 + 1u : t0;
        e.x = 0xffffu | ((t0 + 1u < ntok_first ? 2u : 1u) << 16);
        e.y = (t0 << 16) | (t1 << 24);
    } else if (((e.x >> 16) & 255u) < 2u) {
        e.y = (e.y & 0x00ff00ffu) * 0x101u;            // a lone token: its twin computes the same and is not stored
    }
    const uint32_t expert = e.x & 0xffffu, cnt = (e.x >> 16) & 255u, tok0 = (e.y >> 16) & 255u, tok1 = e.y >> 24;
    REDHIP_STAMP(1);                                   // the pass entry is here
    const uint32_t k0 = sh ? K : (e.y & 255u), k1 = sh ? K : ((e.y >> 8) & 255u);
    float *out0 = a.partial + ((uint64_t)(tok0 * (K + 1u) + k0) * FG + g) * H, *out1 = a.partial + ((uint64_t)(tok1 * (K + 1u) + k1) * FG + g) * H;

    if constexpr (MIX != 0) {
        if (sh) {      // the shared expert's slice from dense f32 data: SwiGLU of the 32 columns, then their part of every output row
            if (tid < 64u) {
                const uint32_t t = tid >> 5, c = tid & 31u;
                const float *gu = a.shared_gu + (uint64_t)(t ? tok1 : tok0) * 2u * F + 32u * g + c;
                const float gv = gu[0], uv = gu[F];
                part[tid] = (gv / (1.0f + expf(-gv))) * uv;
            }
            __syncthreads();
            // Eight lanes per output row, each lane four of the 32 columns for both tokens: a wave-wide load reads the 128-byte slices of
            // eight consecutive rows whole (a lane pair per row, 16 columns each, touched 32 cache lines per load instruction)
            const uint32_t sub = tid & 7u;
            const float4 av = *reinterpret_cast<const float4 *>(part + 4u * sub), bv = *reinterpret_cast<const float4 *>(part + 32u + 4u * sub);
            const float s0 = a.scalar[tok0], s1 = a.scalar[tok1];
            constexpr uint32_t kRows = (uint32_t)NW * 8u;      // rows per round of the workgroup
            for (uint32_t h0 = tid >> 3; h0 < H; h0 += 4u * kRows) {      // four rounds' loads in flight
                float4 w4[4];
#pragma unroll
                for (uint32_t i = 0; i < 4u; ++i) {
                    const uint32_t h = h0 + i * kRows;
                    w4[i] = *reinterpret_cast<const float4 *>(a.shared_dense + (uint64_t)(h < H ? h : h0) * F + 32u * g + 4u * sub);
                }
#pragma unroll
                for (uint32_t i = 0; i < 4u; ++i) {
                    const uint32_t h = h0 + i * kRows;
                    float acc0 = fmaf(w4[i].w, av.w, fmaf(w4[i].z, av.z, fmaf(w4[i].y, av.y, w4[i].x * av.x)));
                    float acc1 = fmaf(w4[i].w, bv.w, fmaf(w4[i].z, bv.z, fmaf(w4[i].y, bv.y, w4[i].x * bv.x)));
#pragma unroll
                    for (int o = 1; o < 8; o <<= 1) { acc0 += __shfl_xor(acc0, o, 64); acc1 += __shfl_xor(acc1, o, 64); }
                    if (h < H) {
                        if (sub == 0u) out0[h] = acc0 * s0;
                        else if (sub == 1u && cnt > 1u) out1[h] = acc1 * s1;
                    }
                }
            }
            return;
        }
    }

    const uint32_t kc = wave % NKC, q0 = wave / NKC;
    const uint32_t G = 16u * kc + blk;
    half4_t ax[8];
    {
        const uint32_t t = (j >> 1) ? tok1 : tok0;
        const _Float16 *src = ((j & 1u) ? a.xl : a.xh) + (uint64_t)t * H + 32u * G;
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) ax[s8] = *reinterpret_cast<const half4_t *>(src + 4 * s8);
    }
    const uint8_t *ex = sh ? a.shared : a.experts + (uint64_t)expert * a.stride;
    const uint8_t *dn = sh ? a.shared_down_cm : a.down_cm + (uint64_t)expert * a.down_stride;
    const uint64_t gate_sc = (uint64_t)F * HG * 8u + (uint64_t)F * HB * 2u;       // IQ2_XS: the scale bytes [row][group] behind qs and ds
    const uint64_t gate_bytes = gate_sc + (MIX == 2 ? (uint64_t)F * HG : 0u);
    uint2 wq[UPW];
    uint32_t wd[UPW];                                    // block scale d (fp16 bits); IQ2_XS: the group's scale byte above it
#pragma unroll
    for (int u = 0; u < UPW; ++u) {
        const uint32_t quad = q0 + (NW / NKC) * u;
        const uint32_t r = 32u * g + 4u * (quad & 7u) + j;
        const uint8_t *mat = ex + (quad < 8u ? 0u : gate_bytes);         // (the same in every lane of the wave; a matrix is far below 4 GB: 32-bit offsets)
        wq[u] = *reinterpret_cast<const uint2 *>(mat + (r * HG + G) * 8u);
        wd[u] = *reinterpret_cast<const uint16_t *>(mat + (F * HG * 8u + (r * HB + (G >> 3)) * 2u));
        if constexpr (MIX == 2) wd[u] |= (uint32_t)mat[(uint32_t)gate_sc + r * HG + G] << 16;
    }
    using DownGroup = typename std::conditional<MIX == 1, uint4, uint2>::type;      // one row's 32 weights of the slice
    const uint8_t *down_qs = dn + (MIX == 1 ? 0u : g * H * (uint32_t)sizeof(DownGroup));
    const uint8_t *down_ds = dn + (FG * H * (uint32_t)sizeof(DownGroup) + (g >> 3) * H * 2u);
    const uint8_t *down_sc = dn + (FG * H * 8u + (FG >> 3) * H * 2u + g * H);      // MIX 2
    DownGroup dq[DU];
    uint32_t dd[DU];                                     // as wd
#pragma unroll
    for (int kk = 0; kk < DU; ++kk) {
        const uint32_t unit = wave + NW * kk;
        const uint32_t r = 64u * (unit < 8u * NKC ? unit : 0u) + lane;
        dq[kk] = *reinterpret_cast<const DownGroup *>(down_qs + (MIX == 1 ? (uint32_t)iq3s_sliced_index(g, r, FG, H) : r) * (uint32_t)sizeof(DownGroup));
        dd[kk] = *reinterpret_cast<const uint16_t *>(down_ds + r * 2u);
        if constexpr (MIX == 2) dd[kk] |= (uint32_t)down_sc[r] << 16;
    }
    if constexpr (MIX == 1) build_iq3s_quads_from(iq3_tab, tid, seed_q3);
    const float w0 = sh ? a.scalar[tok0] : a.weights[tok0 * K + k0], w1 = sh ? a.scalar[tok1] : a.weights[tok1 * K + k1];
    // (an IQ1_M weight is d (2 s + 1) (entry +- 1/8): no 1 / 8)
    const float xs0 = (MIX == 3 ? 1.0f : 0.125f) * exp2i(a.xexp[tok0]), xs1 = (MIX == 3 ? 1.0f : 0.125f) * exp2i(a.xexp[tok1]);
    if constexpr (MIX >= 2) build_codebook_table_from<FMT>(lds, tid, seed_cb);
    else {
        build_tables_rep_from<REP, 16, SREP>(lds, strip, wave, lane, seed_mag);
        reinterpret_cast<uint32_t *>(sign_lut)[tid] = seed_sign;
    }
    const LaneTables lt = lane_tables<REP, kBatchLut>(lds, sign_lut, lane);
    REDHIP_STAMP(2);                                   // loads requested, tables written
    lds_barrier();                                   // tables
    REDHIP_STAMP(3);

    float va[UPW], vb[UPW];
#pragma unroll
    for (int u = 0; u < UPW; ++u) {
        if constexpr (MIX >= 2) group_dot_fmt2<FMT>(wq[u], wd[u] >> 16, ax, lds, va[u], vb[u]);
        else group_dot2_lut<REP, kBatchLut>(wq[u], ax, lt, va[u], vb[u]);
        const float d = scale_to_f32(wd[u]);
        va[u] *= d;
        vb[u] *= d;
    }
    const float ta = quad_column_reduce<UPW>(va, lane), tb = quad_column_reduce<UPW>(vb, lane);
    REDHIP_STAMP(4);                                   // gate / up rows of wave 0 multiplied
    if (reduced_writer<UPW>(lane)) {
        const uint32_t quad = q0 + (NW / NKC) * reduced_unit<UPW>(lane);
        part[kc * 64u + 4u * quad + j] = ta;
        part[NKC * 64u + kc * 64u + 4u * quad + j] = tb;
    }
    lds_barrier();
    REDHIP_STAMP(5);                                   // ... of every wave
    if (tid < 64u) {
        const uint32_t t = tid >> 5, c = tid & 31u;
        const float *pt = part + t * NKC * 64u;
        float gsum = 0.0f, usum = 0.0f;
#pragma unroll
        for (int kk = 0; kk < NKC; ++kk) { gsum += pt[kk * 64 + c]; usum += pt[kk * 64 + 32 + c]; }
        const float xs = t ? xs1 : xs0;
        gsum *= xs;
        usum *= xs;
        const float act = (gsum / (1.0f + expf(-gsum))) * usum;
        float amax = fabsf(act);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        const int ee = prescale_exp(amax);
        split_hi_lo(act, exp2i(-ee), act_hl + t * 64u + c, act_hl + t * 64u + 32u + c);
        if (c == 0u) act_scale[t] = exp2i(ee);
    }
    lds_barrier();
    REDHIP_STAMP(6);                                   // activations exchanged
    half4_t ad[8];
    {
        const _Float16 *src = act_hl + (j >> 1) * 64u + (j & 1u) * 32u;
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) ad[s8] = *reinterpret_cast<const half4_t *>(src + 4 * s8);
    }
    // (an IQ3_S weight is d (1 + 2 nibble) grid byte, an IQ1_M weight as above: no 1 / 8)
    const float post0 = act_scale[0] * w0 * (MIX == 1 || MIX == 3 ? 1.0f : 0.125f), post1 = act_scale[1] * w1 * (MIX == 1 || MIX == 3 ? 1.0f : 0.125f);
#pragma unroll
    for (int kk = 0; kk < DU; ++kk) {
        const uint32_t unit = wave + NW * kk;
        if (unit < 8u * NKC) {
            float da, db;
            if constexpr (MIX == 1) iq3s_group_dot(dq[kk], ad, iq3_tab, da, db);
            else if constexpr (MIX >= 2) group_dot_fmt2<FMT>(dq[kk], dd[kk] >> 16, ad, lds, da, db);
            else group_dot2_lut<REP, kBatchLut>(dq[kk], ad, lt, da, db);
            const float d = scale_to_f32(dd[kk]);
            out0[64u * unit + lane] = da * d * post0;
            if (cnt > 1u) out1[64u * unit + lane] = db * d * post1;
        }
    }
    REDHIP_STAMP(7);                                   // down slice of wave 0 multiplied, stores issued
}

constexpr int kSliceRep = 16;
template <int MIX = 0> constexpr size_t slice_lds_bytes(int nkc) {
    return (size_t)slice_table_bytes<kSliceRep, MIX>() + (size_t)nkc * 64u * 4u + 128u + 16u + sizeof(SelectOut) + (MIX == 1 ? kIq3TableBytes : 0u);
}

hipError_t launch_expert_slices(const void *experts, uint64_t stride, const void *down_cm, uint64_t down_stride, const void *shared, const void *shared_down_cm,
                                const float *logits, const uint32_t *ids_in, const float *weights_in, const float *scalar_in, uint32_t *ids_out,
                                float *weights_out, float *scalar_out, const void *xh, const void *xl, const int *xexp, float *partial, float *out,
                                uint32_t hidden, uint32_t ffn, uint32_t n_expert, uint32_t top_k, hipStream_t s, const float *shared_gu, const float *shared_dense,
                                uint32_t stream_type, const int8_t *grid) {
    if (!fused_iq2_supported(hidden, ffn) || top_k + 1u > (uint32_t)kWaves || n_expert > 1024u || hidden % 32u) return hipErrorInvalidValue;
    if (!logits && (!ids_in || !weights_in || !scalar_in)) return hipErrorInvalidValue;
    const bool mix = shared_gu != nullptr;             // down slices of another format (column-sliced) and the dense shared expert
    if (mix && (!shared_dense || ffn % 256u)) return hipErrorInvalidValue;
    // 1: IQ2_XXS gate / up with IQ3_S words; 2 / 3: IQ2_XS / IQ1_M streams throughout
    const int kind = !mix ? 0 : stream_type == T_IQ2_XS ? 2 : stream_type == T_IQ1_M ? 3 : 1;
    if (kind >= 2 && !grid) return hipErrorInvalidValue;
    const SliceArgs a{static_cast<const uint8_t *>(experts), stride, static_cast<const uint8_t *>(down_cm), down_stride, static_cast<const uint8_t *>(shared),
                      static_cast<const uint8_t *>(shared_down_cm), logits, ids_in, weights_in, scalar_in, ids_out, weights_out, scalar_out,
                      static_cast<const _Float16 *>(xh), static_cast<const _Float16 *>(xl), xexp, partial, hidden, ffn, n_expert, top_k, route_guard().status,
                      nullptr, 0u, nullptr, nullptr, 0u, shared_gu, shared_dense, grid};
    const dim3 grid_dim(ffn / 32u, top_k + (mix ? kSliceSharedParts : 1u));
#define REDHIP_SLICE_MIX(NKC, MIX)                                                                                                     \
    do {                                                                                                                               \
        static bool attr = false;                                                                                                       \
        const size_t dyn = slice_lds_bytes<MIX>(NKC);                                                                                \
        if (!attr) {                                                                                                                    \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(expert_slice_kernel<NKC, kSliceRep, false, MIX>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn); \
            if (e != hipSuccess) return e;                                                                                              \
            attr = true;                                                                                                                \
        }                                                                                                                               \
        REDHIP_LAUNCH((expert_slice_kernel<NKC, kSliceRep, false, MIX>), grid_dim, dim3(kWaves * 64), dyn, s, (const void *)a.logits, a.n_expert, a.top_k, (const void *)a.xh, (const void *)a.xl, 0u, a.hidden, a.ffn, a); \
    } while (0)
#define REDHIP_SLICE(NKC)                                                                                                              \
    do {                                                                                                                               \
        if (kind == 3) REDHIP_SLICE_MIX(NKC, 3); else if (kind == 2) REDHIP_SLICE_MIX(NKC, 2); else if (kind == 1) REDHIP_SLICE_MIX(NKC, 1); else REDHIP_SLICE_MIX(NKC, 0); \
    } while (0)
    prof_set_stage(ST_FUSED_EXPERTS);
    switch (hidden / 512u) {
        case 1: REDHIP_SLICE(1); break;
        case 2: REDHIP_SLICE(2); break;
        case 4: REDHIP_SLICE(4); break;
        case 8: REDHIP_SLICE(8); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_SLICE
#undef REDHIP_SLICE_MIX
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    prof_set_stage(ST_SLICE_SUM);
    REDHIP_LAUNCH(slice_sum_kernel, dim3(hidden / 32u), dim3(256), 0, s, partial, (top_k + 1u) * (ffn / 32u), hidden, out, block_context().resid_a, block_context().resid_b, SumTail{nullptr, nullptr, nullptr, nullptr});
    return hipGetLastError();
}

// One token over the slots of a pool: slot_table[k] = address of slot k's raw bytes, whose re-laid IQ2_XXS copy lies shadow_off behind.
// Two launches: slices (partial [top_k][ffn / 32][hidden]) and their sum into out (and, with a tail, out = out2 = resid + (sum + shared * scalar)).
hipError_t launch_slot_slices(const uint64_t *slot_table, uint64_t shadow_off, const float *weights, uint32_t top_k, uint32_t hidden, uint32_t ffn,
                              const float *x, const float *x1, uint32_t x_split, float *partial, float *out, const float *tail_resid,
                              const float *tail_shared, const float *tail_scalar, float *tail_out2, hipStream_t s, uint32_t kind, const int8_t *grid) {
    if (!fused_iq2_supported(hidden, ffn) || hidden % 32u || !top_k || top_k > 64u || !slot_table || !weights || !x || !partial || !out) return hipErrorInvalidValue;
    if (kind > 3u || (kind >= 2u && !grid) || (kind != 0u && (hidden > 2048u || ffn % 256u))) return hipErrorInvalidValue;
    SliceArgs a{};
    a.grid = grid;
    a.weights_in = weights;
    a.partial = partial;
    a.hidden = hidden; a.ffn = ffn; a.n_expert = 0u; a.top_k = top_k;
    a.slot_table = slot_table;
    a.shadow_off = shadow_off;
    a.x = x; a.x1 = x1; a.x_split = x_split;
    const dim3 grid_dim(ffn / 32u, top_k);
#define REDHIP_SLOT_SLICE_MIX(NKC, MIX)                                                                                                \
    do {                                                                                                                               \
        static bool attr = false;                                                                                                       \
        const size_t dyn = slice_lds_bytes<MIX>(NKC);                                                                                   \
        if (!attr) {                                                                                                                    \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(expert_slice_kernel<NKC, kSliceRep, true, MIX>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn); \
            if (e != hipSuccess) return e;                                                                                              \
            attr = true;                                                                                                                \
        }                                                                                                                               \
        REDHIP_LAUNCH((expert_slice_kernel<NKC, kSliceRep, true, MIX>), grid_dim, dim3(kWaves * 64), dyn, s, (const void *)a.slot_table, a.n_expert, a.top_k, (const void *)a.x, (const void *)a.x1, a.x_split, a.hidden, a.ffn, a); \
    } while (0)
#define REDHIP_SLOT_SLICE(NKC)                                                                                                         \
    do {                                                                                                                               \
        if (kind == 3u) REDHIP_SLOT_SLICE_MIX(NKC, 3); else if (kind == 2u) REDHIP_SLOT_SLICE_MIX(NKC, 2); else if (kind == 1u) REDHIP_SLOT_SLICE_MIX(NKC, 1); else REDHIP_SLOT_SLICE_MIX(NKC, 0); \
    } while (0)
    prof_set_stage(ST_FUSED_EXPERTS);
    switch (hidden / 512u) {
        case 1: REDHIP_SLOT_SLICE(1); break;
        case 2: REDHIP_SLOT_SLICE(2); break;
        case 4: REDHIP_SLOT_SLICE(4); break;
        case 8: REDHIP_SLOT_SLICE_MIX(8, 0); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_SLOT_SLICE
#undef REDHIP_SLOT_SLICE_MIX
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    prof_set_stage(ST_SLICE_SUM);
    const SumTail tail{tail_resid, tail_shared, tail_scalar, tail_out2};
    REDHIP_LAUNCH(slice_sum_kernel, dim3(hidden / 32u), dim3(256), 0, s, partial, top_k * (ffn / 32u), hidden, out, nullptr, nullptr, tail);
    return hipGetLastError();
}

hipError_t launch_batch_slices(const void *experts, uint64_t stride, const void *down_cm, uint64_t down_stride, const void *shared, const void *shared_down_cm,
                               const void *pass_list, const uint32_t *n_pass, const float *weights, const float *scalar, const void *xh, const void *xl,
                               const int *xexp, float *partial, float *out, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, hipStream_t s,
                               const float *shared_gu, const float *shared_dense, uint32_t stream_type, const int8_t *grid) {
    if (!fused_iq2_supported(hidden, ffn) || hidden % 32u || !ntok || ntok > kSelectGroupTokens || ntok * top_k > kGroupMaxPairs || !pass_list || !n_pass) return hipErrorInvalidValue;
    const bool mix = shared_gu != nullptr;
    if (mix ? !shared_dense : (!shared || !shared_down_cm)) return hipErrorInvalidValue;
    if (stream_type && ((stream_type != T_IQ2_XS && stream_type != T_IQ1_M) || !grid || !mix)) return hipErrorInvalidValue;
    const int kind = stream_type == T_IQ2_XS ? 2 : stream_type == T_IQ1_M ? 3 : mix ? 1 : 0;
    const BatchSliceArgs a{static_cast<const uint8_t *>(experts), stride, static_cast<const uint8_t *>(down_cm), down_stride, static_cast<const uint8_t *>(shared),
                           static_cast<const uint8_t *>(shared_down_cm), static_cast<const uint2 *>(pass_list), n_pass, weights, scalar,
                           static_cast<const _Float16 *>(xh), static_cast<const _Float16 *>(xl), xexp, partial, hidden, ffn, top_k, ntok, shared_gu, shared_dense, grid};
    const dim3 grid_dim(ffn / 32u, ntok * top_k + (ntok + 1u) / 2u);      // every pair a pass of its own at most, then the shared expert's passes
#define REDHIP_BSLICE_ONE(NKC, MIX)                                                                                                    \
    do {                                                                                                                               \
        static bool attr = false;                                                                                                       \
        const size_t dyn = (size_t)batch_slice_table_bytes<kBatchRep, MIX>() + (size_t)2u * NKC * 64u * 4u + 256u + 16u + (MIX == 1 ? kIq3TableBytes : 0u); \
        if (!attr) {                                                                                                                    \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(batch_slice_kernel<NKC, kBatchRep, MIX>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn); \
            if (e != hipSuccess) return e;                                                                                              \
            attr = true;                                                                                                                \
        }                                                                                                                               \
        REDHIP_LAUNCH((batch_slice_kernel<NKC, kBatchRep, MIX>), grid_dim, dim3(kWaves * 64), dyn, s, a.pass_list, a.n_pass, a.ntok, a.top_k, a); \
    } while (0)
#define REDHIP_BSLICE(NKC)                                                                                                             \
    do {                                                                                                                               \
        if (kind == 3) REDHIP_BSLICE_ONE(NKC, 3); else if (kind == 2) REDHIP_BSLICE_ONE(NKC, 2); else if (kind == 1) REDHIP_BSLICE_ONE(NKC, 1); else REDHIP_BSLICE_ONE(NKC, 0); \
    } while (0)
    prof_set_stage(ST_FUSED_EXPERTS);
    switch (hidden / 512u) {
        case 1: REDHIP_BSLICE(1); break;
        case 2: REDHIP_BSLICE(2); break;
        case 4: REDHIP_BSLICE(4); break;
        default: return hipErrorInvalidValue;      // (hidden 4096 would spill registers: such layers take their batches on other kernels)
    }
#undef REDHIP_BSLICE
#undef REDHIP_BSLICE_ONE
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    prof_set_stage(ST_SLICE_SUM);
    REDHIP_LAUNCH(slice_sum_kernel, dim3(hidden / 32u, ntok), dim3(256), 0, s, partial, (top_k + 1u) * (ffn / 32u), hidden, out, block_context().resid_a, block_context().resid_b, SumTail{nullptr, nullptr, nullptr, nullptr});
    return hipGetLastError();
}

// One row of a dense f32 matrix against an activation vector kept as fp16 halves + one exponent per 32 columns: the LPR lanes that
// share a row take every LPR-th float4 and meet by butterfly adds. Returns the row's product in every one of those lanes.
template <uint32_t LPR>
__device__ __forceinline__ float dense_row_dot(const float *row, const _Float16 *ah, const _Float16 *al, const int *aexp, uint32_t F, uint32_t part) {
    float acc = 0.0f;
    for (uint32_t c0 = part; c0 < F / 4u; c0 += 8u * LPR) {      // eight float4 per lane and round, all requested before the first is used
        float4 w[8];
        uint2 hv[8], lv[8];
        int ev[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t cr = c0 + LPR * (uint32_t)i, c4 = cr < F / 4u ? cr : F / 4u - 1u;
            w[i] = reinterpret_cast<const float4 *>(row)[c4];
            if (cr >= F / 4u) w[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            hv[i] = reinterpret_cast<const uint2 *>(ah)[c4];
            lv[i] = reinterpret_cast<const uint2 *>(al)[c4];
            ev[i] = aexp[c4 >> 3];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            union { uint2 u; _Float16 h[4]; } hh, ll;
            hh.u = hv[i];
            ll.u = lv[i];
            float t = w[i].x * fmaf((float)ll.h[0], 4.8828125e-4f, (float)hh.h[0]);
            t = fmaf(w[i].y, fmaf((float)ll.h[1], 4.8828125e-4f, (float)hh.h[1]), t);
            t = fmaf(w[i].z, fmaf((float)ll.h[2], 4.8828125e-4f, (float)hh.h[2]), t);
            t = fmaf(w[i].w, fmaf((float)ll.h[3], 4.8828125e-4f, (float)hh.h[3]), t);
            acc = fmaf(t, exp2i(ev[i]), acc);
        }
    }
#pragma unroll
    for (uint32_t o = 1u; o < LPR; o <<= 1) acc += __shfl_xor(acc, (int)o, 64);
    return acc;
}

// The waves behind the routed ones (wave >= top_k of NW) share the shared expert's 8 output rows, read from its dense f32 copy
// [hidden][ffn]; the activations are slot top_k of act_h / act_l / act_exp. Row sums go to part[top_k * 8 + row].
template <int NW>
__device__ __forceinline__ void shared_rows_dense(const float *shared, uint32_t row0, uint32_t F, uint32_t top_k, const _Float16 *act_h, const _Float16 *act_l,
                                                  const int *act_exp, uint32_t wave, uint32_t lane, float *part) {
    const uint32_t spare = (uint32_t)NW - top_k, k = top_k, sw = wave - top_k;
    const _Float16 *ah = act_h + (uint64_t)k * F, *al = act_l + (uint64_t)k * F;
    const int *ae = act_exp + k * (F / 32u);
    if (spare >= 4u) {
        if (sw < 4u) {
            const uint32_t row = 2u * sw + (lane >> 5);
            const float r = dense_row_dot<32>(shared + (uint64_t)(row0 + row) * F, ah, al, ae, F, lane & 31u);
            if ((lane & 31u) == 0u) part[k * 8u + row] = r;
        }
    } else if (spare >= 2u) {
        if (sw < 2u) {
            const uint32_t row = 4u * sw + (lane >> 4);
            const float r = dense_row_dot<16>(shared + (uint64_t)(row0 + row) * F, ah, al, ae, F, lane & 15u);
            if ((lane & 15u) == 0u) part[k * 8u + row] = r;
        }
    } else if (sw == 0u) {
        const uint32_t row = lane >> 3;
        const float r = dense_row_dot<8>(shared + (uint64_t)(row0 + row) * F, ah, al, ae, F, lane & 7u);
        if ((lane & 7u) == 0u) part[k * 8u + row] = r;
    }
}

// Down + combine when the down matrices are not IQ2_XXS (mixed-precision layouts: IQ3_S routed, Q6_K shared): same
// 8 output rows per workgroup, wave = slot, lane = (32-column chunk, row); weights
// decoded from the raw GGUF rows and multiplied in f32 against the activation rebuilt from its fp16 halves.
struct DownRawArgs {
    const uint8_t *experts;    // expert e's raw down rows at experts + e * stride
    uint64_t stride;
    const uint8_t *shared;     // raw down rows of the shared expert
    const uint32_t *ids;
    const float *weights, *scalar;
    const _Float16 *act_h, *act_l;
    const int *act_exp;
    float *out;
    uint32_t hidden, ffn, top_k;
    const float *resid_a, *resid_b;
    const int8_t *grid;        // the caller's codebook of the routed down format (IQ2_XS, IQ1_M) or nullptr
    const float *shared_dense; // when set: the shared expert's down matrix as dense f32 [hidden][ffn], read instead of `shared`
    uint32_t id_limit;         // ids are clamped to id_limit - 1 (RouteGuard)
};

template <uint32_t T>
__device__ __forceinline__ float chunk_dot(const uint8_t *row, uint32_t chunk, const float *av, const int8_t *grid = nullptr) {
    if constexpr (T == T_Q6_K) {
        float sx0 = 0.0f, sx1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) { sx0 += av[i]; sx1 += av[16 + i]; }
        return q6k_dot32(row, chunk, av, sx0, sx1);
    }
    float w[32];
    decode32_cb<T>(row, chunk, w, grid);
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) acc = fmaf(w[i], av[i], acc);
    return acc;
}

template <uint32_t TD, uint32_t TS, int NW>      // NW waves: 12 when the slots fit (a third more registers per lane: no spills), else 16
__global__ __launch_bounds__(NW * 64) void down_combine_raw_kernel(DownRawArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t raw_rows[];     // [slot][8 rows of the slot's matrix]
    __shared__ float part[17 * 8];
    constexpr uint32_t kGridBytes = Codebook<TD>::kBytes;                  // routed format's codebook, copied to LDS (the shared expert never has one)
    __shared__ __attribute__((aligned(16))) int8_t cb[kGridBytes ? kGridBytes : 16u];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    const uint32_t F = a.ffn, FG = F / 32u, FB = F / 256u, n_slot = a.top_k + 1u;
    uint4 cb0 = make_uint4(0u, 0u, 0u, 0u), cb1 = cb0;   // requested first, stored once the wave's rows are on their way
    if constexpr (kGridBytes != 0u) {
        if (tid < kGridBytes / 16u) cb0 = reinterpret_cast<const uint4 *>(a.grid)[tid];
        if (tid + NW * 64u < kGridBytes / 16u) cb1 = reinterpret_cast<const uint4 *>(a.grid)[tid + NW * 64u];
    }
    if (const uint32_t tok = blockIdx.y) {             // several tokens in one launch
        const uint64_t t = tok;
        a.ids += t * a.top_k;
        a.weights += t * a.top_k;
        a.scalar += t;
        a.act_h += t * n_slot * F;
        a.act_l += t * n_slot * F;
        a.act_exp += t * n_slot * FG;
        a.out += t * a.hidden;
        if (a.resid_a) { a.resid_a += t * a.hidden; a.resid_b += t * a.hidden; }
    }
    const uint32_t row0 = 8u * blockIdx.x;
    constexpr uint32_t kMaxBlock = Fmt<TD>::kBlock > Fmt<TS>::kBlock ? Fmt<TD>::kBlock : Fmt<TS>::kBlock;
    const bool is_shared = wave == a.top_k;
    const uint32_t row_bytes = FB * (is_shared ? Fmt<TS>::kBlock : Fmt<TD>::kBlock);
    uint8_t *mine = raw_rows + wave * 8u * FB * kMaxBlock;
    const uint32_t n_raw = a.shared_dense ? a.top_k : n_slot;      // slots decoded from staged raw rows
    if (a.shared_dense && wave >= a.top_k) shared_rows_dense<NW>(a.shared_dense, row0, F, a.top_k, a.act_h, a.act_l, a.act_exp, wave, lane, part);
    if (wave < n_raw) {
        const uint8_t *rows = (is_shared ? a.shared : a.experts + (uint64_t)guarded_id(a.ids[wave], a.id_limit, nullptr) * a.stride) + (uint64_t)row0 * row_bytes;
        wave_stage(mine, rows, 8u * row_bytes, lane);          // 8 rows x FB blocks of 56 .. 210 bytes: a multiple of 16
    }
    if constexpr (kGridBytes != 0u) {
        if (tid < kGridBytes / 16u) reinterpret_cast<uint4 *>(cb)[tid] = cb0;
        if (tid + NW * 64u < kGridBytes / 16u) reinterpret_cast<uint4 *>(cb)[tid + NW * 64u] = cb1;
        __syncthreads();
    }
    if (wave < n_raw) {
        float tot[2] = {0.0f, 0.0f};
        for (uint32_t G = blk; G < FG; G += 16u) {
            float av[32];
            const float sc = exp2i(a.act_exp[wave * FG + G]);
            const uint4 *ph = reinterpret_cast<const uint4 *>(a.act_h + (uint64_t)wave * F + 32u * G), *pl = reinterpret_cast<const uint4 *>(a.act_l + (uint64_t)wave * F + 32u * G);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                union { uint4 u; _Float16 h[8]; } hh, ll;
                hh.u = ph[v];
                ll.u = pl[v];
#pragma unroll
                for (int i = 0; i < 8; ++i) av[8 * v + i] = fmaf((float)ll.h[i], 4.8828125e-4f, (float)hh.h[i]) * sc;
            }
            if (G == blk) wave_lds_sync();                       // the staged rows are visible to the whole wave
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const uint8_t *row = mine + (4u * q + j) * row_bytes;
                tot[q] += is_shared ? chunk_dot<TS>(row, G, av) : chunk_dot<TD>(row, G, av, cb);
            }
        }
        const float r = quad_column_reduce<2>(tot, lane);
        if (reduced_writer<2>(lane)) part[wave * 8u + 4u * reduced_unit<2>(lane) + j] = r;
    }
    __syncthreads();
    if (tid < 8u) {
        float sum = 0.0f;
        for (uint32_t s = 0; s < a.top_k; ++s) sum = fmaf(a.weights[s], part[s * 8u + tid], sum);
        sum = fmaf(a.scalar[0], part[a.top_k * 8u + tid], sum);
        a.out[row0 + tid] = a.resid_a ? (a.resid_a[row0 + tid] + a.resid_b[row0 + tid]) + sum : sum;
    }
}

template <uint32_t TD>
static hipError_t launch_down_raw_shared(uint32_t ts, const DownRawArgs &a, uint32_t ntok, hipStream_t s) {
    const bool narrow = a.top_k + 1u <= 12u;
    const dim3 grid(a.hidden / 8u, ntok), block(narrow ? 12 * 64 : kWaves * 64);
    const size_t lds = (size_t)(a.top_k + 1u) * 8u * (a.ffn / 256u) * 210u;       // sized for the largest block type; at most 17 x 8 x 4 x 210 bytes
#define REDHIP_DRAW(TSV) do { if (narrow) REDHIP_LAUNCH((down_combine_raw_kernel<TD, TSV, 12>), grid, block, lds, s, a); else REDHIP_LAUNCH((down_combine_raw_kernel<TD, TSV, kWaves>), grid, block, lds, s, a); } while (0)
    switch (ts) {
        case T_IQ2_XXS: REDHIP_DRAW(T_IQ2_XXS); break;
        case T_IQ3_S: REDHIP_DRAW(T_IQ3_S); break;
        case T_Q6_K: REDHIP_DRAW(T_Q6_K); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_DRAW
    return hipGetLastError();
}

hipError_t launch_down_combine_raw(uint32_t down_type, uint32_t shared_down_type, const void *experts, uint64_t stride, const void *shared,
                                   const uint32_t *ids, const float *weights, const float *scalar, const void *act_h, const void *act_l,
                                   const int *act_exp, float *out, uint32_t hidden, uint32_t ffn, uint32_t top_k, hipStream_t s, uint32_t ntok,
                                   const int8_t *grid, const float *shared_dense) {
    if (!hidden || hidden % 8u || !ffn || ffn % 256u || top_k + 1u > (uint32_t)kWaves || !ntok || ntok > 65535u) return hipErrorInvalidValue;
    if ((down_type == T_IQ2_XS || down_type == T_IQ1_M) && !grid) return hipErrorInvalidValue;
    const DownRawArgs a{static_cast<const uint8_t *>(experts), stride, static_cast<const uint8_t *>(shared), ids, weights, scalar,
                        static_cast<const _Float16 *>(act_h), static_cast<const _Float16 *>(act_l), act_exp, out, hidden, ffn, top_k,
                        block_context().resid_a, block_context().resid_b, grid, shared_dense, route_guard().id_limit};
    switch (down_type) {
        case T_IQ2_XXS: return launch_down_raw_shared<T_IQ2_XXS>(shared_down_type, a, ntok, s);
        case T_IQ3_S: return launch_down_raw_shared<T_IQ3_S>(shared_down_type, a, ntok, s);
        case T_Q6_K: return launch_down_raw_shared<T_Q6_K>(shared_down_type, a, ntok, s);
        case T_IQ2_XS: return launch_down_raw_shared<T_IQ2_XS>(shared_down_type, a, ntok, s);
        case T_IQ1_M: return launch_down_raw_shared<T_IQ1_M>(shared_down_type, a, ntok, s);
        default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------- IQ3_S down matrices of mixed layouts on the matrix units
//
// "Word-packed IQ3_S" (built at upload): one 32-bit word per eight weights - two 9-bit grid indices (the qh bit folded in) in bits 0-8
// and 9-17, the eight sign bits in 18-25, the group's scale nibble in 26-29 - as one uint4 per 32 weights, [row][K/32], followed by
// d as fp16 [row][K/256]. 130 bytes per 256 weights instead of 110, every load naturally aligned. A weight is
// sign * grid byte * (2 * nibble + 1) * d: the four grid bytes of an entry come as exact fp16 values from an LDS table (512 x 8 bytes),
// the signs are placed as in the IQ2_XXS kernels, and the same 4x4x4 MFMA multiplies them with the fp16 halves of the activations.

// col_major: the same words stored column-sliced (iq3s_sliced_index; d [K / 256][nrows])
__global__ void repack_iq3s_words_kernel(const uint8_t *raw0, uint64_t raw_stride, uint32_t nrows, uint32_t K, uint8_t *packed0, uint64_t packed_stride, int col_major) {
    const uint32_t groups = K / 32u, blocks = K / 256u;
    const uint8_t *raw = raw0 + (uint64_t)blockIdx.y * raw_stride;
    uint8_t *pk = packed0 + (uint64_t)blockIdx.y * packed_stride;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * groups) return;
    const uint32_t r = (uint32_t)(gid / groups), g = (uint32_t)(gid % groups), sub = g & 7u;
    const uint8_t *bp = raw + ((uint64_t)r * blocks + (g >> 3)) * 110u;
    const uint32_t nib = ((uint32_t)bp[106u + (sub >> 1)] >> (4u * (sub & 1u))) & 15u, qh = bp[66u + sub];
    uint32_t w[4];
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t ia = (uint32_t)bp[2u + 8u * sub + 2u * l] | ((qh << (8u - 2u * l)) & 256u);
        const uint32_t ib = (uint32_t)bp[3u + 8u * sub + 2u * l] | ((qh << (7u - 2u * l)) & 256u);
        w[l] = ia | (ib << 9) | ((uint32_t)bp[74u + 4u * sub + l] << 18) | (nib << 26);
    }
    reinterpret_cast<uint4 *>(pk)[col_major ? iq3s_sliced_index(g, r, groups, nrows) : gid] = make_uint4(w[0], w[1], w[2], w[3]);
    if (sub == 0u) reinterpret_cast<uint16_t *>(pk + (uint64_t)nrows * groups * 16u)[col_major ? (uint64_t)(g >> 3) * nrows + r : (uint64_t)r * blocks + (g >> 3)] = (uint16_t)ld_u16(bp);
}

hipError_t launch_repack_iq3s_words(const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K, void *packed, uint64_t packed_stride, hipStream_t s, bool col_major) {
    if (!nrows || !K || K % 256u || !count || count > 65535u) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    REDHIP_LAUNCH(repack_iq3s_words_kernel, dim3((uint32_t)((total + 255u) / 256u), count), dim3(256), 0, s, static_cast<const uint8_t *>(raw), raw_stride, nrows, K,
                  static_cast<uint8_t *>(packed), packed_stride, col_major ? 1 : 0);
    return hipGetLastError();
}

// parity tap: f32 dequantisation from the words, arithmetic as decode32<T_IQ3_S>
__global__ void dequant_iq3s_words_kernel(const uint8_t *pk, uint32_t nrows, uint32_t K, float *out, int col_major) {
    const uint32_t groups = K / 32u, blocks = K / 256u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * groups) return;
    const uint32_t r = (uint32_t)(gid / groups), g = (uint32_t)(gid % groups);
    const uint4 v = reinterpret_cast<const uint4 *>(pk)[col_major ? iq3s_sliced_index(g, r, groups, nrows) : gid];
    const float d = half_bits_to_f32(reinterpret_cast<const uint16_t *>(pk + (uint64_t)nrows * groups * 16u)[col_major ? (uint64_t)(g >> 3) * nrows + r : (uint64_t)r * blocks + (g >> 3)]);
    const float db = d * (float)(1u + 2u * ((v.x >> 26) & 15u));
    const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
    float *o = out + (uint64_t)r * K + 32u * g;
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t wa = redhip_iq3s_grid[w4[l] & 511u], wb = redhip_iq3s_grid[(w4[l] >> 9) & 511u], sg = (w4[l] >> 18) & 255u;
        for (uint32_t j = 0; j < 4u; ++j) {
            o[8u * l + j] = apply_sign(db * (float)((wa >> (8u * j)) & 255u), (sg >> j) & 1u);
            o[8u * l + 4u + j] = apply_sign(db * (float)((wb >> (8u * j)) & 255u), (sg >> (4u + j)) & 1u);
        }
    }
}

hipError_t launch_dequant_iq3s_words(const void *packed, uint32_t nrows, uint32_t K, float *out, hipStream_t s, bool col_major) {
    if (!nrows || !K || K % 256u) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    REDHIP_LAUNCH(dequant_iq3s_words_kernel, dim3((uint32_t)((total + 255u) / 256u)), dim3(256), 0, s, static_cast<const uint8_t *>(packed), nrows, K, out, col_major ? 1 : 0);
    return hipGetLastError();
}

// Down + combine of one token on a mixed layout whose routed down matrices are word-packed IQ3_S: 8 output rows per workgroup, wave s <
// top_k owns the selected expert s (both row quads of the workgroup against all ffn columns), wave top_k the shared expert, read
// from its dense f32 copy [hidden][ffn]. blockIdx.y = token (small batches run one grid layer per token).
struct DownWordsArgs {
    const uint8_t *experts;    // word-packed (IQ3_S) or stream-packed (IQ2_XS, IQ1_M: as their gate / up matrices) down matrix of expert e at experts + e * stride
    uint64_t stride;
    const int8_t *grid;        // the caller's codebook of IQ2_XS / IQ1_M down matrices
    const float *shared;       // dense f32 down matrix of the shared expert
    const uint32_t *ids;
    const float *weights, *scalar;
    const _Float16 *act_h, *act_l;
    const int *act_exp;
    float *out;
    uint32_t hidden, ffn, top_k;
    const float *resid_a, *resid_b;
    uint32_t id_limit;         // ids are clamped to id_limit - 1 (RouteGuard)
};

// FMT: 0 word-packed IQ3_S, 1 stream-packed IQ2_XS, 2 stream-packed IQ1_M; CM (IQ3_S): the words stored column-sliced
// (iq3s_sliced_index, d [ffn / 256][hidden]), the copy that the expert slices of small batches read
template <int NW, int FMT, int CM = 0>
__global__ __launch_bounds__(NW * 64) void down_combine_words_kernel(const uint32_t *ids_first, uint32_t top_k_first, DownWordsArgs a) {
    static_assert(CM == 0 || FMT == 0, "column-sliced copies exist of IQ3_S words only");
    __shared__ __attribute__((aligned(16))) uint8_t lds[FMT == 0 ? kIq3TableBytes : FMT == 1 ? 512u * 16u : 2048u * 16u];
    __shared__ float part[17 * 8];
    const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    // (ids_first, top_k_first repeat a.ids, a.top_k: leading arguments can reach a wave in registers at its start, so the request for
    // the wave's expert id - the head of a chain of three dependent trips - leaves before the argument block has come from memory)
    const uint32_t my_id = wave < top_k_first ? ids_first[blockIdx.y * top_k_first + wave] : 0u;
    const uint32_t F = a.ffn, FG = F / 32u, FB = F / 256u, n_slot = a.top_k + 1u;
    if (const uint32_t tok = blockIdx.y) {
        const uint64_t t = tok;
        a.ids += t * a.top_k;
        a.weights += t * a.top_k;
        a.scalar += t;
        a.act_h += t * n_slot * F;
        a.act_l += t * n_slot * F;
        a.act_exp += t * n_slot * FG;
        a.out += t * a.hidden;
        if (a.resid_a) { a.resid_a += t * a.hidden; a.resid_b += t * a.hidden; }
    }
    const uint32_t row0 = 8u * blockIdx.x;
    const uint32_t n_chunk = (FG + 15u) / 16u;         // ffn <= 1024
    uint4 dq[2][2];            // IQ2_XS / IQ1_M: x, y = the group's uint2, z = the IQ2_XS scale byte
    uint32_t dd[2][2];
    half4_t ax[2][8];
    float sc[2] = {0.0f, 0.0f};
    const bool routed = wave < a.top_k;
    if (routed) {
        const uint8_t *ex = a.experts + (uint64_t)guarded_id(my_id, a.id_limit, nullptr) * a.stride;
        constexpr uint32_t kGroupBytes = FMT == 0 ? 16u : 8u;
        const uint16_t *ds = reinterpret_cast<const uint16_t *>(ex + (uint64_t)a.hidden * FG * kGroupBytes);      // [hidden][FB]
        const uint8_t *scs = ex + (uint64_t)a.hidden * FG * kGroupBytes + (uint64_t)a.hidden * FB * 2u;           // IQ2_XS: [hidden][FG]
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const uint32_t r = row0 + 4u * q + j, G = 16u * c + blk;
                if ((uint32_t)c < n_chunk && G < FG) {
                    if constexpr (FMT == 0) {
                        dq[q][c] = reinterpret_cast<const uint4 *>(ex)[CM != 0 ? iq3s_sliced_index(G, r, FG, a.hidden) : (uint64_t)r * FG + G];
                    } else {
                        const uint2 v = reinterpret_cast<const uint2 *>(ex)[(uint64_t)r * FG + G];
                        dq[q][c] = make_uint4(v.x, v.y, FMT == 1 ? (uint32_t)scs[(uint64_t)r * FG + G] : 0u, 0u);
                    }
                    dd[q][c] = ds[CM != 0 ? (uint64_t)(G >> 3) * a.hidden + r : (uint64_t)r * FB + (G >> 3)];
                }
            }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint32_t G = 16u * c + blk;
            if ((uint32_t)c < n_chunk && G < FG) {
                load_act_operand(ax[c], a.act_h + (uint64_t)wave * F + 32u * G, a.act_l + (uint64_t)wave * F + 32u * G, j);
                sc[c] = exp2i(a.act_exp[wave * FG + G]);
            }
        }
    } else {
        shared_rows_dense<NW>(a.shared, row0, F, a.top_k, a.act_h, a.act_l, a.act_exp, wave, lane, part);
    }
    if constexpr (FMT == 0) build_iq3s_quads(lds, tid);
    else build_codebook_table<FMT>(lds, tid, a.grid, 0u, (uint32_t)NW * 64u);
    __syncthreads();
    if (routed) {
        float tot[2] = {0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint32_t G = 16u * c + blk;
            if ((uint32_t)c < n_chunk && G < FG) {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    float va, vb;
                    if constexpr (FMT == 0) iq3s_group_dot(dq[q][c], ax[c], lds, va, vb);
                    else va = group_dot_fmt<FMT>(make_uint2(dq[q][c].x, dq[q][c].y), dq[q][c].z, ax[c], lds) * (FMT == 1 ? 0.125f : 1.0f);
                    tot[q] += va * scale_to_f32(dd[q][c]) * sc[c];
                }
            }
        }
        const float r = quad_column_reduce<2>(tot, lane);
        if (reduced_writer<2>(lane)) part[wave * 8u + 4u * reduced_unit<2>(lane) + j] = r;
    }
    __syncthreads();
    if (tid < 8u) {
        float sum = 0.0f;
        for (uint32_t s = 0; s < a.top_k; ++s) sum = fmaf(a.weights[s], part[s * 8u + tid], sum);
        sum = fmaf(a.scalar[0], part[a.top_k * 8u + tid], sum);
        a.out[row0 + tid] = a.resid_a ? (a.resid_a[row0 + tid] + a.resid_b[row0 + tid]) + sum : sum;
    }
}

hipError_t launch_down_combine_words(uint32_t down_type, const int8_t *grid, const void *experts, uint64_t stride, const float *shared_dense, const uint32_t *ids,
                                     const float *weights, const float *scalar, const void *act_h, const void *act_l, const int *act_exp, float *out,
                                     uint32_t hidden, uint32_t ffn, uint32_t top_k, hipStream_t s, uint32_t ntok, bool col_major) {
    if (!hidden || hidden % 8u || !ffn || ffn % 256u || ffn > 1024u || top_k + 1u > (uint32_t)kWaves || !ntok || ntok > 65535u || !shared_dense) return hipErrorInvalidValue;
    if ((down_type == T_IQ2_XS || down_type == T_IQ1_M) && (!grid || col_major)) return hipErrorInvalidValue;
    const DownWordsArgs a{static_cast<const uint8_t *>(experts), stride, grid, shared_dense, ids, weights, scalar, static_cast<const _Float16 *>(act_h),
                          static_cast<const _Float16 *>(act_l), act_exp, out, hidden, ffn, top_k, block_context().resid_a, block_context().resid_b, route_guard().id_limit};
    const dim3 grid_dim(hidden / 8u, ntok);
    const bool narrow = top_k + 1u <= 12u;
#define REDHIP_DCW(FMT, CM)                                                                                          \
    do {                                                                                                             \
        if (narrow) REDHIP_LAUNCH((down_combine_words_kernel<12, FMT, CM>), grid_dim, dim3(12 * 64), 0, s, a.ids, a.top_k, a);       \
        else REDHIP_LAUNCH((down_combine_words_kernel<kWaves, FMT, CM>), grid_dim, dim3(kWaves * 64), 0, s, a.ids, a.top_k, a);      \
    } while (0)
    switch (down_type) {
        case T_IQ3_S: if (col_major) REDHIP_DCW(0, 1); else REDHIP_DCW(0, 0); break;
        case T_IQ2_XS: REDHIP_DCW(1, 0); break;
        case T_IQ1_M: REDHIP_DCW(2, 0); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_DCW
    return hipGetLastError();
}

// ---------------------------------------------------------------- small batches (2..16 tokens): select + group, batched gate/up, batched down

// 32 weights of one group against NTP activation operands, each carrying two tokens (rows 0,1 = hi,lo of the
// first, rows 2,3 of the second): the table lookups are done once, the MFMAs once per token pair. The lookups are
// a separate step so that a caller can have those of several groups in flight before it consumes the first.
__device__ __forceinline__ void group_lookup(uint2 q, const uint8_t *lds, uint4 *m) {
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) m[l] = *reinterpret_cast<const uint4 *>(lds + (((q.x >> (8u * l)) & 255u) << 4));
}
template <int NTP>
__device__ __forceinline__ void group_consume(uint2 q, const uint4 *m, const half4_t (*ax)[8], float *va, float *vb) {
    float4_t acc[NTP];
#pragma unroll
    for (int t = 0; t < NTP; ++t) acc[t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t l = 0; l < 4u; ++l) {
        WeightQuad b0, b1;
        place_signs(m[l], (q.y >> (7u * l)) & 127u, b0, b1);
#pragma unroll
        for (int t = 0; t < NTP; ++t) {
            acc[t] = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[t][2u * l], b0.h, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[t][2u * l + 1u], b1.h, acc[t], 0, 0, 0);
        }
    }
    const float sc = (float)(2u * (q.y >> 28) + 1u);
#pragma unroll
    for (int t = 0; t < NTP; ++t) {
        va[t] = (acc[t][0] + acc[t][1] * 4.8828125e-4f) * sc;
        vb[t] = (acc[t][2] + acc[t][3] * 4.8828125e-4f) * sc;
    }
}
template <int NTP>
__device__ __forceinline__ void group_dot_multi(uint2 q, const half4_t (*ax)[8], const uint8_t *lds, float *va, float *vb) {
    uint4 m[4];
    group_lookup(q, lds, m);
    group_consume<NTP>(q, m, ax, va, vb);
}

// activation operand for two tokens: lanes j = 0,1 carry hi,lo of token a; j = 2,3 of token b (32 values at `off`)
__device__ __forceinline__ void load_act_operand2(half4_t *ax, const _Float16 *hi, const _Float16 *lo, uint64_t row_a, uint64_t row_b,
                                                  bool have_b, uint32_t off, uint32_t j) {
    const _Float16 *src = ((j & 1u) ? lo : hi) + ((j & 2u) ? row_b : row_a) + off;
    const bool live = j < 2u || have_b;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        half4_t v = {(_Float16)0, (_Float16)0, (_Float16)0, (_Float16)0};
        if (live) v = *reinterpret_cast<const half4_t *>(src + 4 * s);
        ax[s] = v;
    }
}

struct BatchArgs {
    const uint8_t *experts;
    uint64_t stride;
    const uint8_t *shared;
    const uint32_t *uid, *expert_start, *pair_token, *n_unique;     // grouping (device)
    const float *pair_weight;
    const uint32_t *tok_pair;
    const float *scalar;           // [ntok]
    const _Float16 *xh, *xl;       // [ntok][hidden]
    const int *xexp;               // [ntok]
    _Float16 *act_h, *act_l;       // [P + ntok][ffn]: routed pairs, then the shared expert's pairs (token t at P + t)
    int *act_exp;                  // [P + ntok][ffn / 32]
    float *out;                    // [ntok][hidden]
    uint32_t hidden, ffn, top_k, ntok;
    const float *resid_a, *resid_b;     // when set: out = (resid_a + resid_b) + layer output, [ntok][hidden] each
    const float *shared_gu;             // shared == nullptr: the shared expert's gate . x and up . x, [ntok][2 ffn] f32, already computed
    const int8_t *grid;                 // the caller's codebook when the gate / up matrices are IQ2_XS / IQ1_M streams
    // selection inside the gate/up kernel: logits [ntok][n_expert + 1] from the router launch; the routing (ids, weights, scalar) and its
    // grouping (uid .. n_unique above) are then outputs of the gate/up kernel, written identically by every workgroup
    BatchSelect sel;
};

// Persistent workgroups walk the units (u, g) = (group of pairs, 32 FFN columns): 32 gate + 32 up rows of the
// group's expert (u >= U: the shared expert, two tokens per group when it is packed) for every token that selected it, NTP token pairs per
// pass. The fp16 halves of all tokens sit in LDS, the routing metadata of the workgroup's units too, and the
// weights of the next unit are requested while the current one is computed.
constexpr int kMaxUnits = 16;      // units per workgroup
constexpr int kMaxTok = 8;         // tokens of a small batch

template <int NKC, int NTP, int FMT = 0>      // FMT: 0 IQ2_XXS, 1 IQ2_XS, 2 IQ1_M streams (the latter two: one token pair per pass, no packed shared expert)
__global__ __launch_bounds__(kWaves * 64) void gateup_batch_kernel(BatchArgs a) {
    constexpr int NW = kWaves;
    constexpr int UPW = 16 * NKC / NW;
    static_assert(FMT == 0 || NTP == 1, "the codebook formats run one token pair per pass");
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];                  // activation planes of all tokens
    __shared__ __attribute__((aligned(16))) uint8_t lds[FMT == 0 ? kMagBytes : FMT == 1 ? 512u * 16u : 2048u * 16u];
    __shared__ float part[2][2 * NTP][NKC * 64];                                   // alternating between passes
    __shared__ uint32_t meta_expert[kMaxUnits], meta_p0[kMaxUnits], meta_n[kMaxUnits];
    __shared__ uint8_t meta_tok[kMaxUnits][kMaxTok];
    __shared__ float tok_scale[kMaxTok];
    __shared__ SelectOut sel[kMaxTok];
    __shared__ uint32_t group_lds[kGroupLdsWords];
    __shared__ uint32_t pass_start[130];                 // [128]: passes in all, [129]: whether any group has more than one
    const uint32_t tid = threadIdx.x, lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t H = a.hidden, F = a.ffn, HG = H / 32u, HB = H / 256u, FG = F / 32u, P = a.ntok * a.top_k;
    const uint64_t grid_entry = FMT == 0 && tid < 256u ? redhip_iq2xxs_grid[tid] : 0ull;
    // x operand in LDS as [piece s of 8 bytes][plane][group], plane = 2 * token + (hi, lo) and one more plane of
    // zeros for lanes without a token: the 64 lanes of a wave read the same piece of consecutive groups, and the
    // plane stride of HG + 8 keeps the hi and lo planes on different banks
    const uint32_t PLS = HG + 8u, ZP = 2u * a.ntok, SS = (ZP + 1u) * PLS;
    uint2 *xs = reinterpret_cast<uint2 *>(dyn);
    // staged by the threads from `first` on (the waves below it select meanwhile, when the kernel selects)
    auto stage_x = [&](uint32_t first) {
        const uint32_t st = tid - first, nst = NW * 64u - first;
        if (st < a.ntok) tok_scale[st] = (FMT == 2 ? 1.0f : 0.125f) * exp2i(a.xexp[st]);
        for (uint32_t i = st; i < a.ntok * H / 8u; i += nst) {
            const uint32_t t = i / (H / 8u), c = i % (H / 8u), at = (2u * (c & 3u)) * SS + 2u * t * PLS + (c >> 2);
            const uint4 vh = reinterpret_cast<const uint4 *>(a.xh)[i], vl = reinterpret_cast<const uint4 *>(a.xl)[i];
            xs[at] = make_uint2(vh.x, vh.y);
            xs[at + SS] = make_uint2(vh.z, vh.w);
            xs[at + PLS] = make_uint2(vl.x, vl.y);
            xs[at + PLS + SS] = make_uint2(vl.z, vl.w);
        }
        for (uint32_t i = st; i < 8u * PLS; i += nst) xs[(i / PLS) * SS + ZP * PLS + i % PLS] = make_uint2(0u, 0u);
        if constexpr (FMT != 0) build_codebook_table<FMT>(lds, tid, a.grid, first, nst);
    };
    if (a.sel.logits) {
        // Every workgroup selects and groups for itself (wave t the experts of token t), in place of a launch of its
        // own, and writes the same routing and grouping to device memory: the barrier behind it makes the workgroup's own writes visible
        // to its reads below, and another workgroup's writes carry the same values.
        const uint32_t E = a.sel.n_expert, K = a.top_k;
        if (wave < a.ntok) {
            const float *l = a.sel.logits + (uint64_t)wave * (E + 1u);
            if (E <= 512u) wave_select_topk<8>(l, E, K, &sel[wave]); else wave_select_topk<16>(l, E, K, &sel[wave]);
            wave_lds_sync();
            if (lane < K) { a.sel.ids[wave * K + lane] = sel[wave].ids[lane]; a.sel.weights[wave * K + lane] = sel[wave].w[lane]; }
            if (lane == 0u) a.sel.scalar[wave] = sel[wave].scalar;
        } else {
            stage_x(a.ntok * 64u);
        }
        __syncthreads();
        const GroupJob gj{nullptr, nullptr, a.ntok, K, E, const_cast<uint32_t *>(a.uid), const_cast<uint32_t *>(a.expert_start), const_cast<uint32_t *>(a.pair_token),
                          const_cast<float *>(a.pair_weight), const_cast<uint32_t *>(a.tok_pair), const_cast<uint32_t *>(a.n_unique)};
        group_small(gj, group_lds, [&](uint32_t t, uint32_t k) { return sel[t].ids[k]; }, [&](uint32_t t, uint32_t k) { return sel[t].w[k]; });
        __syncthreads();
    }
    // a packed shared expert is split into groups of two tokens (one pass each) so that no workgroup gets a unit of ntok / 2 passes
    const uint32_t S = a.shared ? (a.ntok + 1u) / 2u : 1u;
    // Routed groups too are scheduled pass by pass (2 * NTP tokens of one expert): pass_start[u] = passes of the groups before u, so
    // that a popular expert's tokens spread over workgroups instead of making one unit of several passes.
    const uint32_t U = a.n_unique[0];
    if (wave == 0u) {                                    // at most 128 groups: two per lane, prefix sums by lane shifts
        constexpr uint32_t TPP = 2u * NTP;
        const uint32_t u0 = lane, u1 = lane + 64u;
        const uint32_t c0 = u0 < U ? (a.expert_start[u0 + 1u] - a.expert_start[u0] + TPP - 1u) / TPP : 0u;
        const uint32_t c1 = u1 < U ? (a.expert_start[u1 + 1u] - a.expert_start[u1] + TPP - 1u) / TPP : 0u;
        if (__ballot(c0 > 1u || c1 > 1u) == 0ull) {      // every group is one pass (the usual case without popular experts): pass = group
            pass_start[u0] = u0 < U ? u0 : U;
            pass_start[u1] = u1 < U ? u1 : U;
            if (lane == 63u) { pass_start[128] = U; pass_start[129] = 0u; }
        } else {
            uint32_t s0 = c0, s1 = c1;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const uint32_t n0 = __shfl_up(s0, o, 64), n1 = __shfl_up(s1, o, 64);
                if (lane >= (uint32_t)o) { s0 += n0; s1 += n1; }
            }
            const uint32_t half = __shfl(s0, 63, 64);
            pass_start[u0] = s0 - c0;
            pass_start[u1] = half + s1 - c1;
            if (lane == 63u) { pass_start[128] = half + s1; pass_start[129] = 1u; }
        }
    }
    __syncthreads();
    const uint32_t V = pass_start[128], n_units = (V + S) * FG;
    uint32_t count = 0u;
    if (blockIdx.x < n_units) count = (n_units - blockIdx.x + gridDim.x - 1u) / gridDim.x;
    if (count > (uint32_t)kMaxUnits) count = kMaxUnits;
    if (count == 0u) return;
    if (tid < count) {
        const uint32_t v = (blockIdx.x + tid * gridDim.x) / FG;      // pass number: routed passes, then the shared expert's
        const bool sh = v >= V;
        uint32_t u = sh ? 0u : v;                        // the group of pass v: the last one with pass_start[u] <= v
        if (pass_start[129]) {
            u = 0u;
#pragma unroll
            for (uint32_t step = 64u; step > 0u; step >>= 1) { if (u + step < U && pass_start[u + step] <= v) u += step; }
        }
        meta_expert[tid] = sh ? 0xffffffffu : a.uid[u];
        const uint32_t sp0 = P + (a.shared ? 2u * (v - V) : 0u), sp1 = a.shared && sp0 + 2u < P + a.ntok ? sp0 + 2u : P + a.ntok;
        const uint32_t rp0 = sh ? 0u : a.expert_start[u] + 2u * NTP * (v - pass_start[u]), rend = sh ? 0u : a.expert_start[u + 1u];
        const uint32_t p0 = sh ? sp0 : rp0, p1 = sh ? sp1 : (rp0 + 2u * NTP < rend ? rp0 + 2u * NTP : rend);
        meta_p0[tid] = p0;
        meta_n[tid] = sh && !a.shared ? 0u : p1 - p0;      // a shared expert that is not packed has no passes: its products are an input
        for (uint32_t i = 0; i < p1 - p0 && i < (uint32_t)kMaxTok; ++i) meta_tok[tid][i] = (uint8_t)(sh ? p0 - P + i : a.pair_token[p0 + i]);
    }
    if (!a.sel.logits) stage_x(0u);
    if constexpr (FMT == 0) build_tables(lds, tid, grid_entry);
    __syncthreads();

    const uint64_t qs_bytes = (uint64_t)F * HG * 8u, sc_off = qs_bytes + (uint64_t)F * HB * 2u, gate_bytes = sc_off + (FMT == 1 ? (uint64_t)F * HG : 0u);
    const uint32_t kc = wave % NKC, q0 = wave / NKC;              // wave-uniform: they stay in scalar registers
    const uint32_t G = 16u * kc + blk;
    const uint32_t lane_q = (j * HG + blk) * 8u, lane_d = (j * HB + (blk >> 3)) * 2u;
    uint2 wq[UPW], wq_next[UPW];
    uint32_t wd[UPW], wd_next[UPW];               // bits 0-15: d; IQ2_XS: bits 16-23 the group's scale byte
    // uniform row base + one lane offset for all units of the wave
    auto load_weights = [&](uint32_t k, uint2 *q, uint32_t *d) {
        const uint32_t g = (blockIdx.x + k * gridDim.x) % FG;
        const uint32_t e = __builtin_amdgcn_readfirstlane(meta_expert[k]);
        const uint8_t *ex = e == 0xffffffffu ? (a.shared ? a.shared : a.experts) : a.experts + (uint64_t)e * a.stride;   // (never-used weights of a unit without passes)
#pragma unroll
        for (int un = 0; un < UPW; ++un) {
            const uint32_t quad = q0 + (NW / NKC) * un;
            const uint32_t row = 32u * g + 4u * (quad & 7u);
            const uint8_t *mat = ex + (quad < 8u ? 0u : gate_bytes);
            q[un] = *reinterpret_cast<const uint2 *>(mat + ((uint64_t)row * HG + 16u * kc) * 8u + lane_q);
            d[un] = *reinterpret_cast<const uint16_t *>(mat + qs_bytes + ((uint64_t)row * HB + 2u * kc) * 2u + lane_d);
            if constexpr (FMT == 1) d[un] |= (uint32_t)(mat + sc_off)[(uint64_t)row * HG + 16u * kc + (lane_q >> 3)] << 16;
        }
    };
    load_weights(0u, wq, wd);
    uint32_t pass = 0u;
    for (uint32_t k = 0; k < count; ++k) {
        // always issued (the last unit asks for its own weights again): a conditional request would make the
        // compiler wait for it before the first use of the current weights
        load_weights(k + 1u < count ? k + 1u : k, wq_next, wd_next);
        const uint32_t g = (blockIdx.x + k * gridDim.x) % FG, n = meta_n[k], p0 = meta_p0[k];
        for (uint32_t pp = 0; pp < n; pp += 2u * NTP, ++pass) {
            float (*pbuf)[NKC * 64] = part[pass & 1u];
            half4_t ax[NTP][8];
#pragma unroll
            for (int t = 0; t < NTP; ++t) {
                const uint32_t ip = pp + 2u * t + (j >> 1);
                const uint32_t plane = ip < n ? 2u * meta_tok[k][ip] + (j & 1u) : ZP;
                const uint2 *src = xs + plane * PLS + G;
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    union { uint2 u; half4_t h; } v4;
                    v4.u = src[(uint32_t)s * SS];
                    ax[t][s] = v4.h;
                }
            }
            float v[2 * NTP][UPW];
            // one lookup round trip costs far more than its issue slot: the table reads run kAhead groups ahead
            constexpr int kAhead = UPW < 2 ? UPW : 2;
            uint4 m[UPW][4];
            uint2 q[UPW];
#pragma unroll
            for (int un = 0; un < UPW; ++un) {
                q[un] = wq[un];
                asm volatile("" : "+v"(q[un].x), "+v"(q[un].y));   // table addresses are formed here, not hoisted out of the pass loop
            }
            if constexpr (FMT == 0) {
#pragma unroll
                for (int un = 0; un < kAhead; ++un) group_lookup(q[un], lds, m[un]);
            }
#pragma unroll
            for (int un = 0; un < UPW; ++un) {
                float va[NTP], vb[NTP];
                if constexpr (FMT == 0) {
                    if (un + kAhead < UPW) group_lookup(q[un + kAhead], lds, m[un + kAhead]);
                    group_consume<NTP>(q[un], m[un], ax, va, vb);
                } else {
                    group_dot_fmt2<FMT>(q[un], wd[un] >> 16, ax[0], lds, va[0], vb[0]);
                }
                const float d = scale_to_f32(wd[un] & 0xffffu);
#pragma unroll
                for (int t = 0; t < NTP; ++t) { v[2 * t][un] = va[t] * d; v[2 * t + 1][un] = vb[t] * d; }
            }
#pragma unroll
            for (int t = 0; t < 2 * NTP; ++t) {
                const float tot = quad_column_reduce<UPW>(v[t], lane);
                if (reduced_writer<UPW>(lane)) pbuf[t][kc * 64u + 4u * (q0 + (NW / NKC) * reduced_unit<UPW>(lane)) + j] = tot;
            }
            // the only barrier of a pass: the next pass writes the other half of `part`, and the one after that
            // comes behind the next barrier, which the lanes below reach only after they have read this half
            __syncthreads();
            if (tid < 32u * 2u * NTP) {
                const uint32_t t = tid >> 5, c = tid & 31u, ip = pp + t;
                if (ip < n) {
                    float gsum = 0.0f, usum = 0.0f;
#pragma unroll
                    for (int kk = 0; kk < NKC; ++kk) { gsum += pbuf[t][kk * 64 + c]; usum += pbuf[t][kk * 64 + 32 + c]; }
                    const float xs = tok_scale[meta_tok[k][ip]];
                    gsum *= xs;
                    usum *= xs;
                    const float act = (gsum / (1.0f + expf(-gsum))) * usum;
                    float amax = fabsf(act);
#pragma unroll
                    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
                    const int e = prescale_exp(amax);
                    const uint64_t pr = p0 + ip;
                    split_hi_lo(act, exp2i(-e), a.act_h + pr * F + 32u * g + c, a.act_l + pr * F + 32u * g + c);
                    if (c == 0u) a.act_exp[pr * FG + g] = e;
                }
            }
        }
        if (!a.shared && meta_expert[k] == 0xffffffffu && tid < 32u * a.ntok) {      // SwiGLU of the given products, token t at pair P + t
            const uint32_t t = tid >> 5, c = tid & 31u;
            const float gsum = a.shared_gu[(uint64_t)t * 2u * F + 32u * g + c], usum = a.shared_gu[(uint64_t)t * 2u * F + F + 32u * g + c];
            const float act = (gsum / (1.0f + expf(-gsum))) * usum;
            float amax = fabsf(act);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const int e = prescale_exp(amax);
            const uint64_t pr = P + t;
            split_hi_lo(act, exp2i(-e), a.act_h + pr * F + 32u * g + c, a.act_l + pr * F + 32u * g + c);
            if (c == 0u) a.act_exp[pr * FG + g] = e;
        }
#pragma unroll
        for (int un = 0; un < UPW; ++un) { wq[un] = wq_next[un]; wd[un] = wd_next[un]; }
    }
}

struct BatchWordsArgs {
    const uint8_t *experts;    // packed down matrix of expert e at experts + e * stride
    uint64_t stride;
    const int8_t *grid;        // the caller's codebook (IQ2_XS / IQ1_M)
    const float *shared;       // dense f32 [hidden][ffn]
    const uint32_t *uid, *expert_start, *n_unique;
    const float *pair_weight;
    const uint32_t *tok_pair;
    const float *scalar;
    const _Float16 *act_h, *act_l;
    const int *act_exp;
    float *out;
    uint32_t hidden, ffn, top_k, ntok;
    const float *resid_a, *resid_b;
};

template <int MAXPAIR, int NCH, int GPW, int FMT>     // GPW: groups of a wave whose weights are in registers at once
__global__ __launch_bounds__(kWaves * 64) void down_batch_words_kernel(BatchWordsArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[FMT == 0 ? kIq3TableBytes : FMT == 1 ? 512u * 16u : 2048u * 16u];
    __shared__ float part[MAXPAIR * 8];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t H = a.hidden, F = a.ffn, FG = F / 32u, FB = F / 256u, P = a.ntok * a.top_k;
    const uint32_t row0 = 8u * blockIdx.x, U = __builtin_amdgcn_readfirstlane(a.n_unique[0]);
    const uint64_t qs_bytes = (uint64_t)H * FG * (FMT == 0 ? 16u : 8u), sc_off = qs_bytes + (uint64_t)H * FB * 2u;      // IQ2_XS: scale bytes [hidden][FG] behind d

    uint4 wq[GPW][NCH][2];
    uint32_t wd[GPW][NCH], gp0[GPW], gp1[GPW];      // wd: the two rows' block scales, 16 bits each
    // metadata and weights of groups first, first + 16, ...; indices are clamped so that every request is valid
    auto request = [&](uint32_t first) {
#pragma unroll
        for (int i = 0; i < GPW; ++i) {
            const uint32_t u = first + 16u * (uint32_t)i, uc = u < U ? u : U - 1u;      // routed groups only (U >= 1)
            // wave-uniform values: kept in scalar registers
            const uint32_t e = __builtin_amdgcn_readfirstlane(a.uid[uc]), es0 = __builtin_amdgcn_readfirstlane(a.expert_start[uc]),
                           es1 = __builtin_amdgcn_readfirstlane(a.expert_start[uc + 1u]);
            gp0[i] = es0;
            gp1[i] = u < U ? es1 : es0;
            const uint8_t *dn = a.experts + (uint64_t)e * a.stride;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const uint32_t G = 16u * (uint32_t)c + blk, Gc = G < FG ? G : FG - 1u;
                uint32_t d2 = 0u;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const uint32_t r = row0 + 4u * (uint32_t)q + j;
                    if constexpr (FMT == 0) {
                        wq[i][c][q] = reinterpret_cast<const uint4 *>(dn)[(uint64_t)r * FG + Gc];
                    } else {
                        const uint2 v = reinterpret_cast<const uint2 *>(dn)[(uint64_t)r * FG + Gc];
                        wq[i][c][q] = make_uint4(v.x, v.y, FMT == 1 ? (uint32_t)(dn + sc_off)[(uint64_t)r * FG + Gc] : 0u, 0u);
                    }
                    d2 |= (uint32_t)reinterpret_cast<const uint16_t *>(dn + qs_bytes)[(uint64_t)r * FB + (Gc >> 3)] << (16 * q);
                }
                wd[i][c] = d2;
            }
        }
    };
    struct Pass { half4_t ax[NCH][8]; float sa[NCH], sb[NCH]; };
    // activations of pairs pp (and pp + 1 if it belongs to the group); pp is clamped into the buffer
    auto load_pass = [&](uint32_t pp, uint32_t p1, Pass &ps) {
        const uint32_t last = P + a.ntok - 1u, pa = pp < last ? pp : last, pb = pa + 1u < p1 ? pa + 1u : pa;
        const bool have_b = pp + 1u < p1;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const uint32_t G = 16u * (uint32_t)c + blk, Gc = G < FG ? G : FG - 1u;
            load_act_operand2(ps.ax[c], a.act_h, a.act_l, (uint64_t)pa * F, (uint64_t)pb * F, true, 32u * Gc, j);
            const float live = G < FG ? 1.0f : 0.0f;
            ps.sa[c] = live * exp2i(a.act_exp[pa * FG + Gc]);
            ps.sb[c] = have_b ? live * exp2i(a.act_exp[pb * FG + Gc]) : 0.0f;
        }
    };
    // the shared expert: its 8 rows from the dense copy; token t on wave 15 - t, before that wave's routed groups take their registers
    if (15u - wave < a.ntok) {
        const uint32_t p = P + (15u - wave), row = lane >> 3;
        const float r = dense_row_dot<8>(a.shared + (uint64_t)(row0 + row) * F, a.act_h + (uint64_t)p * F, a.act_l + (uint64_t)p * F, a.act_exp + p * FG, F, lane & 7u);
        if ((lane & 7u) == 0u) part[p * 8u + row] = r;
    }
    request(wave);
    if constexpr (FMT == 0) build_iq3s_quads(lds, tid);
    else build_codebook_table<FMT>(lds, tid, a.grid, 0u, kWaves * 64u);
    __syncthreads();

    for (uint32_t first = wave; first < U; first += 16u * GPW) {
        if (first != wave) request(first);
        Pass buf[2];                                     // activations of the current and of the next group
        load_pass(gp0[0], gp1[0], buf[0]);
#pragma unroll
        for (int i = 0; i < GPW; ++i) {
            Pass &cur = buf[NCH == 1 ? i & 1 : 0];
            if (NCH == 1 && i + 1 < GPW) load_pass(gp0[i + 1 < GPW ? i + 1 : i], gp1[i + 1 < GPW ? i + 1 : i], buf[(i + 1) & 1]);
            if (NCH != 1 && i > 0) load_pass(gp0[i], gp1[i], cur);
            for (uint32_t pp = gp0[i]; pp < gp1[i]; pp += 2u) {
                if (pp != gp0[i]) load_pass(pp, gp1[i], cur);            // further passes of a large group
                const bool have_b = pp + 1u < gp1[i];
                float tot_a[2] = {0.0f, 0.0f}, tot_b[2] = {0.0f, 0.0f};
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const float d = scale_to_f32(wd[i][c] >> (16 * q));
                        float va, vb;
                        const uint4 w = wq[i][c][q];
                        if constexpr (FMT == 0) iq3s_group_dot(w, cur.ax[c], lds, va, vb);
                        else group_dot_fmt2<FMT>(make_uint2(w.x, w.y), w.z, cur.ax[c], lds, va, vb);
                        tot_a[q] += va * d * cur.sa[c];
                        tot_b[q] += vb * d * cur.sb[c];
                    }
                }
                const float ra = quad_column_reduce<2>(tot_a, lane), rb = quad_column_reduce<2>(tot_b, lane);
                if (reduced_writer<2>(lane)) {
                    const uint32_t rr = 4u * reduced_unit<2>(lane) + j;
                    part[pp * 8u + rr] = ra;
                    if (have_b) part[(pp + 1u) * 8u + rr] = rb;
                }
            }
        }
    }
    __syncthreads();
    for (uint32_t i = tid; i < a.ntok * 8u; i += kWaves * 64u) {
        const uint32_t t = i >> 3, r = i & 7u;
        float sum = 0.0f;
        for (uint32_t k = 0; k < a.top_k; ++k) {
            const uint32_t p = a.tok_pair[t * a.top_k + k];
            sum = fmaf(a.pair_weight[p] * (FMT == 1 ? 0.125f : 1.0f), part[p * 8u + r], sum);      // IQ2_XS: d/8
        }
        sum = fmaf(a.scalar[t], part[(P + t) * 8u + r], sum);
        const uint64_t at = (uint64_t)t * H + row0 + r;
        a.out[at] = a.resid_a ? (a.resid_a[at] + a.resid_b[at]) + sum : sum;
    }
}

// Batched down + combine on raw GGUF rows (mixed layouts): 8 output rows per workgroup, wave w owns
// the groups w, w + 16, ..., the last group is the shared expert with every token) with the decode of down_combine_raw_kernel. A wave
// stages the 8 rows of its group in LDS (the next group's rows are requested into registers before the current group is computed),
// decodes a row's chunk once and applies it to every pair of the group, so a matrix is read once however many tokens selected it.
struct DownBatchRawArgs {
    const uint8_t *experts;    // expert e's raw down rows at experts + e * stride
    uint64_t stride;
    const uint8_t *shared;     // raw down rows of the shared expert
    const uint32_t *uid, *expert_start, *n_unique;
    const float *pair_weight;
    const uint32_t *tok_pair;
    const float *scalar;
    const _Float16 *act_h, *act_l;     // [P + ntok][ffn]
    const int *act_exp;
    float *out;
    uint32_t hidden, ffn, top_k, ntok;
    const float *resid_a, *resid_b;
};

template <uint32_t TD, uint32_t TS>
__global__ __launch_bounds__(kWaves * 64) void down_batch_raw_kernel(DownBatchRawArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t raw_rows[];     // [wave][8 rows of the wave's current group]
    __shared__ float part[144 * 8];
    constexpr uint32_t kMaxBlock = Fmt<TD>::kBlock > Fmt<TS>::kBlock ? Fmt<TD>::kBlock : Fmt<TS>::kBlock;
    constexpr int kVec = 5;                            // 16-byte pieces per lane of one group's rows: 8 rows x 3 blocks x 210 bytes at most
    const uint32_t tid = threadIdx.x, lane = tid & 63u, blk = lane >> 2, j = lane & 3u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t H = a.hidden, F = a.ffn, FG = F / 32u, FB = F / 256u, P = a.ntok * a.top_k;
    const uint32_t row0 = 8u * blockIdx.x, U = __builtin_amdgcn_readfirstlane(a.n_unique[0]);
    uint8_t *mine = raw_rows + wave * 8u * FB * kMaxBlock;
    uint4 nxt[kVec];
    auto fetch = [&](uint32_t u) {                      // rows of group u (clamped: the last request repeats the shared expert's)
        const uint32_t uc = u < U ? u : U;
        const bool sh = uc == U;
        const uint32_t row_bytes = FB * (sh ? Fmt<TS>::kBlock : Fmt<TD>::kBlock), nvec = 8u * row_bytes / 16u;
        const uint32_t e = __builtin_amdgcn_readfirstlane(a.uid[sh ? 0u : uc]);
        const uint4 *src = reinterpret_cast<const uint4 *>((sh ? a.shared : a.experts + (uint64_t)e * a.stride) + (uint64_t)row0 * row_bytes);
#pragma unroll
        for (int i = 0; i < kVec; ++i) {
            const uint32_t at = lane + 64u * (uint32_t)i;
            nxt[i] = src[at < nvec ? at : nvec - 1u];
        }
    };
    fetch(wave);
    for (uint32_t u = wave; u <= U; u += 16u) {
        const bool sh = u == U;
        const uint32_t row_bytes = FB * (sh ? Fmt<TS>::kBlock : Fmt<TD>::kBlock), nvec = 8u * row_bytes / 16u;
        const uint32_t p0 = sh ? P : __builtin_amdgcn_readfirstlane(a.expert_start[u]);
        const uint32_t p1 = sh ? P + a.ntok : __builtin_amdgcn_readfirstlane(a.expert_start[u + 1u]);
        wave_lds_sync();                               // the previous group's reads of `mine` are done
#pragma unroll
        for (int i = 0; i < kVec; ++i) {
            const uint32_t at = lane + 64u * (uint32_t)i;
            if (at < nvec) reinterpret_cast<uint4 *>(mine)[at] = nxt[i];
        }
        fetch(u + 16u);                                // always issued: a conditional request would be waited for at once
        wave_lds_sync();
        for (uint32_t G = blk; G < FG; G += 16u) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                float w[32];
                const uint8_t *row = mine + (4u * (uint32_t)q + j) * row_bytes;
                if (sh) decode32<TS>(row, G, w); else decode32<TD>(row, G, w);
                for (uint32_t p = p0; p < p1; ++p) {
                    const float sc = exp2i(a.act_exp[p * FG + G]);
                    const uint4 *ph = reinterpret_cast<const uint4 *>(a.act_h + (uint64_t)p * F + 32u * G), *pl = reinterpret_cast<const uint4 *>(a.act_l + (uint64_t)p * F + 32u * G);
                    float acc = 0.0f;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        union { uint4 u; _Float16 h[8]; } hh, ll;
                        hh.u = ph[v];
                        ll.u = pl[v];
#pragma unroll
                        for (int i = 0; i < 8; ++i) acc = fmaf(w[8 * v + i], fmaf((float)ll.h[i], 4.8828125e-4f, (float)hh.h[i]), acc);
                    }
                    acc *= sc;
                    const float r = quad_column_reduce<1>(&acc, lane);      // over the 16 lanes that share j (one chunk each)
                    if (reduced_writer<1>(lane)) {
                        float *dst = &part[p * 8u + 4u * (uint32_t)q + j];
                        *dst = G == blk ? r : *dst + r;
                    }
                }
            }
        }
    }
    __syncthreads();
    for (uint32_t i = tid; i < a.ntok * 8u; i += kWaves * 64u) {
        const uint32_t t = i >> 3, r = i & 7u;
        float sum = 0.0f;
        for (uint32_t k = 0; k < a.top_k; ++k) {
            const uint32_t p = a.tok_pair[t * a.top_k + k];
            sum = fmaf(a.pair_weight[p], part[p * 8u + r], sum);
        }
        sum = fmaf(a.scalar[t], part[(P + t) * 8u + r], sum);
        const uint64_t at = (uint64_t)t * H + row0 + r;
        a.out[at] = a.resid_a ? (a.resid_a[at] + a.resid_b[at]) + sum : sum;
    }
}

static hipError_t launch_gateup_batch_kernel(const BatchArgs &a, uint32_t n_groups, hipStream_t s, uint32_t gate_up_type = T_IQ2_XXS);
static bool batch_select_ok(const BatchSelect &b, uint32_t ntok, uint32_t top_k, uint32_t n_expert) {
    return b.logits && b.ids && b.weights && b.scalar && b.n_expert == n_expert && n_expert <= 1024u && top_k <= 16u && top_k <= n_expert && ntok * top_k <= 128u;
}

template <uint32_t TD>
static hipError_t launch_down_batch_raw_shared(uint32_t ts, const DownBatchRawArgs &a, hipStream_t s) {
    const dim3 grid(a.hidden / 8u), block(kWaves * 64);
    const size_t lds = (size_t)kWaves * 8u * (a.ffn / 256u) * 210u;       // sized for the largest block type: 53,760 bytes at ffn 512
#define REDHIP_DBR(TSV)                                                                                                     \
    do {                                                                                                                    \
        static bool attr = false;                                                                                            \
        if (!attr) {                                                                                                         \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(down_batch_raw_kernel<TD, TSV>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); \
            if (e != hipSuccess) return e;                                                                                   \
            attr = true;                                                                                                     \
        }                                                                                                                    \
        REDHIP_LAUNCH((down_batch_raw_kernel<TD, TSV>), grid, block, lds, s, a);                                              \
    } while (0)
    switch (ts) {
        case T_IQ2_XXS: REDHIP_DBR(T_IQ2_XXS); break;
        case T_IQ3_S: REDHIP_DBR(T_IQ3_S); break;
        case T_Q6_K: REDHIP_DBR(T_Q6_K); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_DBR
    return hipGetLastError();
}

// Small batch on a mixed layout, pairs grouped by expert: packed IQ2_XXS gate/up matrices on the batched MFMA kernel (the shared
// expert's gate / up products come in as shared_gu [ntok][2 ffn]), raw down matrices of any built-in type on the batched raw-row kernel.
hipError_t launch_batch_mixed(uint32_t gate_up_type, const int8_t *gate_up_grid, const void *packed, uint64_t packed_stride, const float *shared_gu,
                              uint32_t down_type, const int8_t *down_grid, uint32_t shared_down_type,
                              const void *raw_down, uint64_t raw_stride, const void *shared_down, const void *words_down, uint64_t words_stride,
                              const float *dense_down, const uint32_t *uid, const uint32_t *expert_start,
                              const uint32_t *pair_token, const uint32_t *n_unique, const float *pair_weight, const uint32_t *tok_pair,
                              const float *scalar, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l, int *act_exp,
                              float *out, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert, hipStream_t s,
                              const BatchSelect *select) {
    if (!fused_iq2_supported(hidden, ffn) || !ntok || ntok > (uint32_t)kMaxTok || ntok * top_k + ntok > 144u || !shared_gu) return hipErrorInvalidValue;
    const bool gu_codebook = gate_up_type == T_IQ2_XS || gate_up_type == T_IQ1_M, dn_codebook = down_type == T_IQ2_XS || down_type == T_IQ1_M;
    if ((gate_up_type != T_IQ2_XXS && !gu_codebook) || (gu_codebook && !gate_up_grid) || (dn_codebook && !down_grid)) return hipErrorInvalidValue;
    const bool on_mfma = words_down && dense_down && (down_type == T_IQ3_S || dn_codebook);
    if (!on_mfma) {                                    // the staged raw rows move in 16-byte pieces, five per lane at most
        if (ffn > 768u) return hipErrorInvalidValue;
        const uint32_t rbd = (ffn / 256u) * block_bytes(down_type), rbs = (ffn / 256u) * block_bytes(shared_down_type);
        if (!rbd || !rbs || (8u * rbd) % 16u || (8u * rbs) % 16u || raw_stride % 16u || (uintptr_t)raw_down % 16u || (uintptr_t)shared_down % 16u) return hipErrorInvalidValue;
    }
    BatchArgs a{static_cast<const uint8_t *>(packed), packed_stride, nullptr, uid, expert_start, pair_token, n_unique,
                pair_weight, tok_pair, scalar, static_cast<const _Float16 *>(xh), static_cast<const _Float16 *>(xl), xexp,
                static_cast<_Float16 *>(act_h), static_cast<_Float16 *>(act_l), act_exp, out, hidden, ffn, top_k, ntok,
                nullptr, nullptr, shared_gu, gate_up_grid, BatchSelect{}};
    if (select && !batch_select_ok(*select, ntok, top_k, n_expert)) return hipErrorInvalidValue;
    if (select) a.sel = *select;
    const uint32_t P = ntok * top_k, n_groups = (P < n_expert ? P : n_expert) + 1u;
    hipError_t e = launch_gateup_batch_kernel(a, (P + (P < n_expert ? P : n_expert) + 1u) / 2u + 1u, s, gate_up_type);      // passes of two tokens + the shared expert's SwiGLU unit
    if (e != hipSuccess) return e;
    prof_set_stage(ST_BATCH_DOWN);
    if (on_mfma) {      // packed down matrices on the matrix units, the shared expert's rows from its f32 copy
        const BatchWordsArgs w{static_cast<const uint8_t *>(words_down), words_stride, down_grid, dense_down, uid, expert_start, n_unique, pair_weight, tok_pair, scalar,
                               static_cast<const _Float16 *>(act_h), static_cast<const _Float16 *>(act_l), act_exp, out, hidden, ffn, top_k, ntok,
                               block_context().resid_a, block_context().resid_b};
        const uint32_t groups_per_wave = (n_groups + kWaves - 1u) / kWaves;
        const dim3 dgrid(hidden / 8u), dblock(kWaves * 64);
        // (at most three groups of a wave in flight: IQ3_S words take twice the registers of the IQ2_XXS groups)
#define REDHIP_DBW(FMT)                                                                                                          \
    do {                                                                                                                         \
        if (ffn > 512u) REDHIP_LAUNCH((down_batch_words_kernel<144, 2, 1, FMT>), dgrid, dblock, 0, s, w);                         \
        else if (groups_per_wave <= 2u) REDHIP_LAUNCH((down_batch_words_kernel<144, 1, 2, FMT>), dgrid, dblock, 0, s, w);         \
        else REDHIP_LAUNCH((down_batch_words_kernel<144, 1, 3, FMT>), dgrid, dblock, 0, s, w);                                    \
    } while (0)
        switch (down_type) {
            case T_IQ3_S: REDHIP_DBW(0); break;
            case T_IQ2_XS: REDHIP_DBW(1); break;
            default: REDHIP_DBW(2); break;
        }
#undef REDHIP_DBW
        return hipGetLastError();
    }
    const DownBatchRawArgs d{static_cast<const uint8_t *>(raw_down), raw_stride, static_cast<const uint8_t *>(shared_down), uid, expert_start, n_unique,
                             pair_weight, tok_pair, scalar, static_cast<const _Float16 *>(act_h), static_cast<const _Float16 *>(act_l), act_exp, out,
                             hidden, ffn, top_k, ntok, block_context().resid_a, block_context().resid_b};
    switch (down_type) {
        case T_IQ2_XXS: return launch_down_batch_raw_shared<T_IQ2_XXS>(shared_down_type, d, s);
        case T_IQ3_S: return launch_down_batch_raw_shared<T_IQ3_S>(shared_down_type, d, s);
        case T_Q6_K: return launch_down_batch_raw_shared<T_Q6_K>(shared_down_type, d, s);
        default: return hipErrorInvalidValue;
    }
}

static hipError_t launch_gateup_batch_kernel(const BatchArgs &a, uint32_t n_groups, hipStream_t s, uint32_t gate_up_type) {
    const uint32_t hidden = a.hidden, ffn = a.ffn, ntok = a.ntok;
    const uint32_t unit_bound = n_groups * (ffn / 32u);
    const dim3 grid(256u * ((unit_bound + 256u * kMaxUnits - 1u) / (256u * kMaxUnits)));
    const size_t dyn_lds = (size_t)(2u * ntok + 1u) * (hidden / 32u + 8u) * 64u;   // hi and lo plane per token + a zero plane, 8 pieces of 8 bytes per group
    const bool codebook = gate_up_type == T_IQ2_XS || gate_up_type == T_IQ1_M;
    if (codebook && (ntok > 8u || a.shared || !a.grid)) return hipErrorInvalidValue;
    prof_set_stage(ST_BATCH_GATEUP);
#define REDHIP_GUB_ONE(NKC, NTP, FMT)                                                                                      \
    do {                                                                                                                  \
        static bool attr = false;                                                                                          \
        if (!attr) {                                                                                                       \
            hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void *>(gateup_batch_kernel<NKC, NTP, FMT>), hipFuncAttributeMaxDynamicSharedMemorySize, (FMT == 2 ? 104 : 128) * 1024); \
            if (e1 != hipSuccess) return e1;                                                                               \
            attr = true;                                                                                                   \
        }                                                                                                                  \
        REDHIP_LAUNCH((gateup_batch_kernel<NKC, NTP, FMT>), grid, dim3(kWaves * 64), dyn_lds, s, a);                        \
    } while (0)
#define REDHIP_GUB(NKC)                                                                                                   \
    do {                                                                                                                  \
        /* two token pairs per pass keep the kernel inside 128 VGPRs; larger groups take more passes */                  \
        if (gate_up_type == T_IQ2_XS) REDHIP_GUB_ONE(NKC, 1, 1);                                                          \
        else if (gate_up_type == T_IQ1_M) REDHIP_GUB_ONE(NKC, 1, 2);                                                      \
        else if (ntok <= 8u) REDHIP_GUB_ONE(NKC, 1, 0);                                                                   \
        else REDHIP_GUB_ONE(NKC, 2, 0);                                                                                   \
    } while (0)
    // (beside the static tables: 51 KB with the IQ1_M codebook, 27 KB otherwise, of 160 KB per workgroup)
    if (dyn_lds > (gate_up_type == T_IQ1_M ? 104u : 128u) * 1024u) return hipErrorInvalidValue;
    switch (hidden / 512u) {
        case 1: REDHIP_GUB(1); break;
        case 2: REDHIP_GUB(2); break;
        case 4: REDHIP_GUB(4); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_GUB
#undef REDHIP_GUB_ONE
    return hipGetLastError();
}


hipError_t launch_gateup_select(const void *experts, uint64_t stride, const void *shared, const void *shared_q6k, const float *x,
                                const float *shared_gu, const float *logits, const uint32_t *ids_in, uint32_t *ids_out, float *weights_out,
                                float *scalar_out, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l, int *act_exp,
                                uint32_t hidden, uint32_t ffn, uint32_t n_expert, uint32_t top_k, hipStream_t s, uint32_t ntok,
                                uint32_t gate_up_type, const int8_t *grid) {
    if (!fused_iq2_supported(hidden, ffn) || (!shared && !shared_gu && (!shared_q6k || !x)) || !ntok || ntok > 64u) return hipErrorInvalidValue;
    const bool codebook = gate_up_type == T_IQ2_XS || gate_up_type == T_IQ1_M;
    if ((gate_up_type != T_IQ2_XXS && !codebook) || (codebook && (!grid || shared))) return hipErrorInvalidValue;
    GateUpArgs a{static_cast<const uint8_t *>(experts), stride, grid, static_cast<const uint8_t *>(shared), static_cast<const uint8_t *>(shared_q6k), x,
                 shared_gu, logits, ids_in, ids_out, weights_out, scalar_out, static_cast<const _Float16 *>(xh), static_cast<const _Float16 *>(xl),
                 xexp, static_cast<_Float16 *>(act_h), static_cast<_Float16 *>(act_l), act_exp, hidden, ffn, n_expert, top_k, route_guard().status};
    const dim3 grid_dim(ffn / 32u, top_k + 1u, ntok);
    const size_t dyn = shared || shared_gu ? 0u : (size_t)64u * (hidden / 256u) * 210u + (size_t)(hidden + hidden / 32u + hidden / 16u) * 4u;   // raw Q6_K rows of one unit of the shared expert, x, sums of 16 x
    const size_t dyn_max = gate_up_type == T_IQ1_M ? 120u * 1024u : 144u * 1024u;      // beside the static decode table (32 KB for IQ1_M)
#define REDHIP_GUS(NKC, FMT)                                                                                                           \
    do {                                                                                                                               \
        static bool attr = false;                                                                                                       \
        if (dyn && !attr) {                                                                                                             \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gateup_select_kernel<NKC, FMT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn_max); \
            if (e != hipSuccess) return e;                                                                                              \
            attr = true;                                                                                                                \
        }                                                                                                                               \
        REDHIP_LAUNCH((gateup_select_kernel<NKC, FMT>), grid_dim, dim3(kWaves * 64), dyn, s, a.logits, a.n_expert, a.top_k, a);           \
    } while (0)
#define REDHIP_GUS_FMT(NKC)                                                                                                            \
    do {                                                                                                                               \
        if (gate_up_type == T_IQ2_XS) REDHIP_GUS(NKC, 1);                                                                               \
        else if (gate_up_type == T_IQ1_M) REDHIP_GUS(NKC, 2);                                                                           \
        else REDHIP_GUS(NKC, 0);                                                                                                        \
    } while (0)
    if (dyn > dyn_max) return hipErrorInvalidValue;
    switch (hidden / 512u) {
        case 1: REDHIP_GUS_FMT(1); break;
        case 2: REDHIP_GUS_FMT(2); break;
        case 4: REDHIP_GUS_FMT(4); break;
        case 8: REDHIP_GUS_FMT(8); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_GUS_FMT
#undef REDHIP_GUS
    return hipGetLastError();
}

}  // namespace redhip

extern "C" int redhip_timeline_read(uint64_t *stamps, uint32_t n_groups, uint32_t clear) {
#ifdef REDHIP_TIMELINE
    if (!stamps || !n_groups || n_groups > redhip::kTimelineGroups) return 0;
    if (hipDeviceSynchronize() != hipSuccess) return 0;
    const size_t bytes = (size_t)n_groups * redhip::kTimelineSlots * sizeof(uint64_t);
    if (hipMemcpyFromSymbol(stamps, HIP_SYMBOL(redhip::g_timeline), bytes) != hipSuccess) return 0;
    if (clear) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(redhip::g_timeline)) != hipSuccess || hipMemset(p, 0, sizeof(uint64_t) * redhip::kTimelineGroups * redhip::kTimelineSlots) != hipSuccess) return 0;
    }
    return 1;
#else
    (void)stamps; (void)n_groups; (void)clear;
    return 0;                                            // this library was built without the phase stamps
#endif
}
