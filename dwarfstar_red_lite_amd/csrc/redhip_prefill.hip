// Prefill chunk (tens to hundreds of tokens) on packed IQ2_XXS experts: the (token, expert) pairs of one expert are cut
// into tiles of 16 pairs, and a tile against 16 weight rows is one v_mfma_f32_16x16x16_f16 per 16 columns.
//
// Operand mapping (lane l, r = l % 16, q = l / 16), checked on gfx950:
//   A[i = r][k = 4q .. 4q + 3]   activations of tile pair r
//   B[k = 4q .. 4q + 3][j = r]   weights of row r
//   D[i = 4q .. 4q + 3][j = r]   the lane receives ITS OWN row against four pairs
// One IQ2_XXS group (32 weights, 4 grid entries) is two MFMAs: lane (r, q) decodes grid entry q of row r and feeds its
// first four weights to the first MFMA and the other four to the second; the activation operand uses the same k order
// (columns 8q .. 8q + 3, then 8q + 4 .. 8q + 7 of the group). Because D's column is the lane's own row, the group scale
// (2 s + 1) and the block scale d are applied to the accumulator, per group, in f32. Activations are fp16 hi + lo
// halves (22 bits) as everywhere else, so a group costs four MFMAs.
//
// Reference behaviour this replaces: native/redmetal_engine_prefill.m:1246-1330 (grouped GEMM over expert slices)
// with the arithmetic of native/redlite_native_reference.c:251-382.
#include <hip/hip_runtime.h>

#include "redhip_mfma.h"

namespace redhip {

constexpr uint32_t kTile = kPrefillTile;         // pairs per tile
constexpr uint32_t kRowPad = 32u;               // fp16 elements of padding per staged activation row (64 B: spreads the rows over the banks)

// ---------------------------------------------------------------- tile list

// the tile lists (TileLists) as a launch of their own, for callers whose pair sort did not write them
constexpr uint32_t kWideTile = kPrefillWideTile;
__global__ __launch_bounds__(1024) void build_tiles_kernel(const uint32_t *expert_start, const uint32_t *n_unique, uint32_t P, TileLists tl) {
    __shared__ uint32_t wave_total[3][16];
    const uint32_t tid = threadIdx.x, U = n_unique[0];
    uint32_t p0 = 0u, n = 0u;
    if (tid < U) { p0 = expert_start[tid]; n = expert_start[tid + 1u] - p0; }
    build_tile_lists(U, p0, n, P, tl, wave_total);
}

struct PrefillArgs {
    const uint8_t *experts;
    uint64_t stride;
    const uint8_t *shared;
    const uint32_t *uid, *pair_token, *n_unique;
    const uint32_t *tile_group, *tile_pair0, *tile_n, *n_tiles;
    const _Float16 *xh, *xl;       // [ntok][hidden]
    const int *xexp;               // [ntok]
    _Float16 *act_h, *act_l;       // [P + ntok][ffn]
    int *act_exp;                  // [P + ntok][ffn / 32]
    float *tmp, *sh_tmp;           // down outputs: [P][hidden] routed pairs, [ntok][hidden] shared expert
    uint32_t hidden, ffn, top_k, ntok;
};

// signed weights of grid entry q of a group word, and the group scale 2 s + 1
__device__ __forceinline__ void decode_entry(uint2 w, uint32_t q, const uint8_t *lds, WeightQuad &b0, WeightQuad &b1) {
    const uint32_t idx = (w.x >> (8u * q)) & 255u, s7 = (w.y >> (7u * q)) & 127u;
    place_signs(*reinterpret_cast<const uint4 *>(lds + (idx << 4)), s7, b0, b1);
}

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
union Half8 { uint4 u; half4_t h[2]; half8_t v; };

// one group of 32 columns: acc = A x B over the group's 32 k, activations hi and lo; returns the four f32 sums of this
// lane's row against pairs 4q .. 4q + 3, without the scales
__device__ __forceinline__ float4_t group_mfma(const Half8 &xa, const Half8 &xb, const WeightQuad &b0, const WeightQuad &b1) {
    float4_t hi = {0.0f, 0.0f, 0.0f, 0.0f}, lo = {0.0f, 0.0f, 0.0f, 0.0f};
    hi = __builtin_amdgcn_mfma_f32_16x16x16f16(xa.h[0], b0.h, hi, 0, 0, 0);
    lo = __builtin_amdgcn_mfma_f32_16x16x16f16(xb.h[0], b0.h, lo, 0, 0, 0);
    hi = __builtin_amdgcn_mfma_f32_16x16x16f16(xa.h[1], b1.h, hi, 0, 0, 0);
    lo = __builtin_amdgcn_mfma_f32_16x16x16f16(xb.h[1], b1.h, lo, 0, 0, 0);
    float4_t r;
#pragma unroll
    for (int t = 0; t < 4; ++t) r[t] = fmaf(lo[t], 4.8828125e-4f, hi[t]);
    return r;
}

// ---------------------------------------------------------------- gate/up + SwiGLU

// A workgroup takes whole tiles: the fp16 halves of the tile's 16 tokens are staged in LDS once, then the 32-column
// groups g of the FFN are walked. Wave = (row tile rt: gate rows 0..15, gate 16..31, up 0..15, up 16..31 of the
// group; K quarter kc). The four K quarters meet in LDS, SwiGLU and the fp16 split of the activation follow.
template <int NKC>          // hidden = 512 * NKC
__global__ __launch_bounds__(kWaves * 64) void prefill_gateup_kernel(PrefillArgs a) {
    constexpr uint32_t H = 512u * NKC, HG = H / 32u, HB = H / 256u, GPW = HG / 4u, ROW = H + kRowPad;   // GPW: groups per wave
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];          // xs_h | xs_l: [16][ROW] fp16
    __shared__ __attribute__((aligned(16))) uint8_t lds[kMagBytes];
    __shared__ float part[4][kTile][68];                   // [K quarter][pair][row of the unit], rows padded off the bank stride
    __shared__ float tok_scale[kTile];
    __shared__ uint32_t tok_of[kTile];
    _Float16 *xs_h = reinterpret_cast<_Float16 *>(dyn), *xs_l = xs_h + kTile * ROW;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), rt = wave & 3u, kc = wave >> 2;
    const uint32_t F = a.ffn, FG = F / 32u, P = a.ntok * a.top_k;
    const uint64_t grid_entry = tid < 256u ? redhip_iq2xxs_grid[tid] : 0ull;
    build_tables(lds, tid, grid_entry);
    const uint32_t T = a.n_tiles[0], U = a.n_unique[0];
    const uint64_t qs_bytes = (uint64_t)F * HG * 8u, gate_bytes = qs_bytes + (uint64_t)F * HB * 2u;

    for (uint32_t tile = blockIdx.x; tile < T; tile += gridDim.x) {
        const uint32_t u = a.tile_group[tile], p0 = a.tile_pair0[tile], n = a.tile_n[tile];
        const uint8_t *ex = u == U ? a.shared : a.experts + (uint64_t)a.uid[u] * a.stride;
        __syncthreads();                                   // the previous tile's readers are done with xs / tok_of
        if (tid < kTile) {
            const uint32_t p = p0 + tid, tok = tid < n ? (p < P ? a.pair_token[p] : p - P) : 0u;
            tok_of[tid] = tok;
            tok_scale[tid] = tid < n ? 0.125f * exp2i(a.xexp[tok]) : 0.0f;
        }
        __syncthreads();
        {   // stage: 64 lanes per token, 16 bytes at a time
            const uint32_t i = tid >> 6, tok = tok_of[i];
            const bool live = i < n;
            for (uint32_t c = lane; c < H / 8u; c += 64u) {
                uint4 vh = make_uint4(0u, 0u, 0u, 0u), vl = vh;
                if (live) {
                    vh = reinterpret_cast<const uint4 *>(a.xh + (uint64_t)tok * H)[c];
                    vl = reinterpret_cast<const uint4 *>(a.xl + (uint64_t)tok * H)[c];
                }
                *reinterpret_cast<uint4 *>(xs_h + i * ROW + 8u * c) = vh;
                *reinterpret_cast<uint4 *>(xs_l + i * ROW + 8u * c) = vl;
            }
        }
        __syncthreads();

        // The wave's weights arrive in chunks of four groups (32 bytes of a row); the chunk after the current one, in
        // the same unit or the next, is always in flight.
        constexpr uint32_t CPU = GPW / 4u;                 // chunks per unit
        const uint8_t *mat = ex + (rt < 2u ? 0u : gate_bytes);
        auto chunk_ptr = [&](uint32_t it) {
            const uint32_t g = it / CPU, c = it % CPU, row = 32u * g + 16u * (rt & 1u) + r;
            return reinterpret_cast<const uint4 *>(mat + ((uint64_t)row * HG + kc * GPW + 4u * c) * 8u);
        };
        auto scale_ptr = [&](uint32_t it) {
            const uint32_t g = it / CPU, c = it % CPU, row = 32u * g + 16u * (rt & 1u) + r;
            return reinterpret_cast<const uint16_t *>(mat + qs_bytes) + (uint64_t)row * HB + (kc * GPW + 4u * c) / 8u;
        };
        const uint32_t n_it = FG * CPU;
        uint4 wa = chunk_ptr(0u)[0], wb = chunk_ptr(0u)[1];
        uint32_t dcur = *scale_ptr(0u);
        float4_t tot = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 1
        for (uint32_t it = 0; it < n_it; ++it) {
            const uint32_t nx = it + 1u < n_it ? it + 1u : it;
            const uint4 na = chunk_ptr(nx)[0], nb = chunk_ptr(nx)[1];
            const uint32_t dnext = *scale_ptr(nx);
            const uint32_t g = it / CPU, c = it % CPU;
            const uint2 w4[4] = {make_uint2(wa.x, wa.y), make_uint2(wa.z, wa.w), make_uint2(wb.x, wb.y), make_uint2(wb.z, wb.w)};
            const uint32_t lane_off = r * ROW + 32u * (kc * GPW + 4u * c) + 8u * q;
            float4_t blk = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) {
                Half8 xa, xb;
                xa.u = *reinterpret_cast<const uint4 *>(xs_h + lane_off + 32u * k);
                xb.u = *reinterpret_cast<const uint4 *>(xs_l + lane_off + 32u * k);
                WeightQuad b0, b1;
                decode_entry(w4[k], q, lds, b0, b1);
                const float4_t sm = group_mfma(xa, xb, b0, b1);
                const float f = (float)(2u * (w4[k].y >> 28) + 1u);
#pragma unroll
                for (int t = 0; t < 4; ++t) blk[t] = fmaf(sm[t], f, blk[t]);
            }
            const float d = scale_to_f32(dcur);
#pragma unroll
            for (int t = 0; t < 4; ++t) tot[t] = fmaf(blk[t], d, tot[t]);
            wa = na; wb = nb; dcur = dnext;
            if (c + 1u < CPU) continue;
            // end of the unit (g): the K quarters meet
#pragma unroll
            for (int t = 0; t < 4; ++t) part[kc][4u * q + (uint32_t)t][16u * rt + r] = tot[t];
            __syncthreads();
            if (tid < 512u) {                              // (pair i, column c): lanes 0..31 of a half wave share a pair
                const uint32_t i = tid >> 5, c = tid & 31u;
                float gsum = 0.0f, usum = 0.0f;
#pragma unroll
                for (int k4 = 0; k4 < 4; ++k4) { gsum += part[k4][i][c]; usum += part[k4][i][32u + c]; }
                const float xs = tok_scale[i];
                gsum *= xs;
                usum *= xs;
                const float act = (gsum / (1.0f + expf(-gsum))) * usum;
                float amax = fabsf(act);
#pragma unroll
                for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
                if (i < n) {
                    const int e = prescale_exp(amax);
                    const uint64_t pr = p0 + i;
                    split_hi_lo(act, exp2i(-e), a.act_h + pr * F + 32u * g + c, a.act_l + pr * F + 32u * g + c);
                    if (c == 0u) a.act_exp[pr * FG + g] = e;
                }
            }
            __syncthreads();
            tot = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
}

// ---------------------------------------------------------------- down

// A workgroup takes whole tiles: the tile's activations (fp16 halves and the per-group exponents) are staged in LDS,
// then wave w computes rows 256 c + 16 w .. + 15 for c = 0, 1, ... against all ffn columns. No reduction across
// waves: every lane ends with its row against four pairs and stores them.
template <int NFG>          // ffn = 32 * NFG
__global__ __launch_bounds__(kWaves * 64) void prefill_down_kernel(PrefillArgs a) {
    constexpr uint32_t F = 32u * NFG, FB = F / 256u, ROW = F + kRowPad;
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];          // as_h | as_l: [16][ROW] fp16
    _Float16 *as_h = reinterpret_cast<_Float16 *>(dyn), *as_l = as_h + kTile * ROW;
    __shared__ __attribute__((aligned(16))) float as_scale[NFG][kTile];     // 2^exponent of (group, pair)
    __shared__ __attribute__((aligned(16))) uint8_t lds[kMagBytes];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t H = a.hidden, P = a.ntok * a.top_k;
    const uint64_t grid_entry = tid < 256u ? redhip_iq2xxs_grid[tid] : 0ull;
    build_tables(lds, tid, grid_entry);
    const uint32_t T = a.n_tiles[0], U = a.n_unique[0];
    const uint64_t down_off = 2u * ((uint64_t)F * (H / 32u) * 8u + (uint64_t)F * (H / 256u) * 2u), qs_bytes = (uint64_t)H * NFG * 8u;

    for (uint32_t tile = blockIdx.x; tile < T; tile += gridDim.x) {
        const uint32_t u = a.tile_group[tile], p0 = a.tile_pair0[tile], n = a.tile_n[tile];
        const uint8_t *dn = (u == U ? a.shared : a.experts + (uint64_t)a.uid[u] * a.stride) + down_off;
        __syncthreads();
        {
            const uint32_t i = tid >> 6;
            const bool live = i < n;
            for (uint32_t c = lane; c < F / 8u; c += 64u) {
                uint4 vh = make_uint4(0u, 0u, 0u, 0u), vl = vh;
                if (live) {
                    vh = reinterpret_cast<const uint4 *>(a.act_h + (uint64_t)(p0 + i) * F)[c];
                    vl = reinterpret_cast<const uint4 *>(a.act_l + (uint64_t)(p0 + i) * F)[c];
                }
                *reinterpret_cast<uint4 *>(as_h + i * ROW + 8u * c) = vh;
                *reinterpret_cast<uint4 *>(as_l + i * ROW + 8u * c) = vl;
            }
            if (lane < NFG) as_scale[lane][i] = live ? exp2i(a.act_exp[(uint64_t)(p0 + i) * NFG + lane]) : 0.0f;
        }
        __syncthreads();
        // Rows 256 b + 16 w + r for b = 0, 1, ...; the weights of a row arrive in chunks of four groups and the chunk after
        // the current one (same row block or the next) is always in flight.
        constexpr uint32_t NCK = NFG / 4u;
        const uint8_t *lane_rows = dn + (uint64_t)(16u * wave + r) * NFG * 8u;
        const uint16_t *lane_ds = reinterpret_cast<const uint16_t *>(dn + qs_bytes) + (uint64_t)(16u * wave + r) * FB;
        auto chunk_ptr = [&](uint32_t it) {
            return reinterpret_cast<const uint4 *>(lane_rows + (uint64_t)(it / NCK) * (16u * kWaves) * NFG * 8u + (it % NCK) * 32u);
        };
        auto scale_ptr = [&](uint32_t it) { return lane_ds + (uint64_t)(it / NCK) * (16u * kWaves) * FB + (it % NCK) / 2u; };
        const uint32_t n_it = (H / (16u * kWaves)) * NCK;
        uint4 wa = chunk_ptr(0u)[0], wb = chunk_ptr(0u)[1];
        uint32_t dcur = *scale_ptr(0u);
        float4_t tot = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 1
        for (uint32_t it = 0; it < n_it; ++it) {
            const uint32_t nx = it + 1u < n_it ? it + 1u : it;
            const uint4 na = chunk_ptr(nx)[0], nb = chunk_ptr(nx)[1];
            const uint32_t dnext = *scale_ptr(nx);
            const uint32_t c = it % NCK;
            const uint2 w4[4] = {make_uint2(wa.x, wa.y), make_uint2(wa.z, wa.w), make_uint2(wb.x, wb.y), make_uint2(wb.z, wb.w)};
            const uint32_t lane_off = r * ROW + 128u * c + 8u * q;
            float4_t blk = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) {
                Half8 xa, xb;
                xa.u = *reinterpret_cast<const uint4 *>(as_h + lane_off + 32u * k);
                xb.u = *reinterpret_cast<const uint4 *>(as_l + lane_off + 32u * k);
                WeightQuad b0, b1;
                decode_entry(w4[k], q, lds, b0, b1);
                const float4_t sm = group_mfma(xa, xb, b0, b1);
                const float4_t sc = *reinterpret_cast<const float4_t *>(&as_scale[4u * c + k][4u * q]);
                const float f = (float)(2u * (w4[k].y >> 28) + 1u);
#pragma unroll
                for (int t = 0; t < 4; ++t) blk[t] = fmaf(sm[t] * sc[t], f, blk[t]);
            }
            const float d = scale_to_f32(dcur);
#pragma unroll
            for (int t = 0; t < 4; ++t) tot[t] = fmaf(blk[t], d, tot[t]);
            wa = na; wb = nb; dcur = dnext;
            if (c + 1u < NCK) continue;
            const uint32_t row = (it / NCK) * (16u * kWaves) + 16u * wave + r;
#pragma unroll
            for (uint32_t t = 0; t < 4u; ++t) {
                const uint32_t i = 4u * q + t, p = p0 + i;
                if (i < n) (p < P ? a.tmp + (uint64_t)p * H : a.sh_tmp + (uint64_t)(p - P) * H)[row] = 0.125f * tot[t];
            }
            tot = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
}

// ---------------------------------------------------------------- register-resident tiles on the tile-major layout (ffn <= 512)

// The two kernels above read a tile's activations from LDS again for every 16 weight rows and gather their weights 16 bytes
// per row. These keep the activations in registers instead: a wave owns a fixed slice of the contraction dimension for the
// whole tile, so the MFMA A operands (fp16 hi and lo halves, 16 bytes each per group of 32 columns) are loaded once per tile.
// The weights come from a second, tile-major copy of the packed matrices in which the 32-byte chunks (four groups) of 16
// consecutive rows lie next to each other, so that one wave-wide load is 512 contiguous bytes:
//   chunk (row, c)  at ((row / 16 * (K / 128) + c) * 16 + row % 16) * 32          c = chunk of four groups along K
//   scale (row, b)  at qs_bytes + ((row / 16 * (K / 256) + b) * 16 + row % 16) * 2
// Decode: a 64 KB LDS table holds the eight fp16 magnitudes of every grid entry times every group scale 2 s + 1 (exact in
// fp16), a 2 KB table the eight sign masks of every 7-bit sign field, so a lane's eight weights are two table reads and four
// XORs, and with the group scale folded into the weights the groups of a chunk accumulate in the matrix units
// (v_mfma_f32_16x16x32_f16: one instruction per group and activation half). The SwiGLU activations of a tile are collected
// in LDS as f32 and split into fp16 halves with one exponent per pair and half of the FFN columns, so the down kernel
// scales its sums once per chunk instead of once per group (22 bits below the largest activation of 256 columns is ample
// for a dot product).
constexpr int kRegWaves = 8;
// The gate/up tile kernel works in items of kItemUnits units of 32 FFN columns (= one 128-column chunk of the down kernels) and leaves
// one activation exponent per pair and item: kExpPerPair ints per pair (ffn <= 512).
constexpr uint32_t kItemUnits = 4u, kExpPerPair = 4u;
constexpr uint32_t kScaledMagBytes = 16u * 256u * 16u;      // [group scale s][grid entry]
constexpr uint32_t kSignBytes = 128u * 16u;                 // [seven sign bits] (the eighth sign is their parity)

// row-major packed matrix -> tile-major copy; one thread per 32-byte chunk, the scales ride along (with_sc: an IQ2_XS stream, whose scale
// bytes [row][group] follow qs and ds; the four of a chunk become one 32-bit word at (tile, chunk, row) like the chunk itself)
__global__ void tile_packed_kernel(const uint8_t *packed, uint64_t packed_stride, uint32_t nrows, uint32_t K, uint8_t *tiled, uint64_t tiled_stride, int with_sc) {
    const uint32_t NC = K / 128u, NB = K / 256u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * NC) return;
    const uint32_t row = (uint32_t)(gid / NC), c = (uint32_t)(gid % NC);
    const uint8_t *src = packed + (uint64_t)blockIdx.y * packed_stride;
    uint8_t *dst = tiled + (uint64_t)blockIdx.y * tiled_stride;
    const uint64_t qs_bytes = (uint64_t)nrows * (K / 32u) * 8u;
    const uint4 *sp = reinterpret_cast<const uint4 *>(src + ((uint64_t)row * (K / 32u) + 4u * c) * 8u);
    uint4 *dp = reinterpret_cast<uint4 *>(dst + (((uint64_t)(row / 16u) * NC + c) * 16u + row % 16u) * 32u);
    dp[0] = sp[0];
    dp[1] = sp[1];
    if ((c & 1u) == 0u) {
        const uint32_t b = c / 2u;
        reinterpret_cast<uint16_t *>(dst + qs_bytes)[((uint64_t)(row / 16u) * NB + b) * 16u + row % 16u] =
            reinterpret_cast<const uint16_t *>(src + qs_bytes)[(uint64_t)row * NB + b];
    }
    if (with_sc) {
        const uint64_t sc_off = qs_bytes + (uint64_t)nrows * NB * 2u;
        reinterpret_cast<uint32_t *>(dst + sc_off)[((uint64_t)(row / 16u) * NC + c) * 16u + row % 16u] =
            *reinterpret_cast<const uint32_t *>(src + sc_off + (uint64_t)row * (K / 32u) + 4u * c);
    }
}

hipError_t launch_tile_packed(const void *packed, uint64_t packed_stride, uint32_t count, uint32_t nrows, uint32_t K, void *tiled, uint64_t tiled_stride,
                              hipStream_t s, bool with_sc) {
    if (!nrows || nrows % 16u || !K || K % 256u || !count || count > 65535u) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 128u);
    REDHIP_LAUNCH(tile_packed_kernel, dim3((uint32_t)((total + 255u) / 256u), count), dim3(256), 0, s, static_cast<const uint8_t *>(packed), packed_stride,
                  nrows, K, static_cast<uint8_t *>(tiled), tiled_stride, with_sc ? 1 : 0);
    return hipGetLastError();
}

// both decode tables, built once per workgroup
__device__ __forceinline__ void build_scaled_tables(uint8_t *mag, uint8_t *sgn, uint32_t tid, uint32_t nthreads) {
    for (uint32_t e = tid; e < 16u * 256u; e += nthreads) {
        const uint64_t grid_entry = redhip_iq2xxs_grid[e & 255u];
        const float f = (float)(2u * (e >> 8) + 1u);
        uint32_t w4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const _Float16 lo = (_Float16)(f * (float)((uint32_t)(grid_entry >> (16 * i)) & 255u)), hi = (_Float16)(f * (float)((uint32_t)(grid_entry >> (16 * i + 8)) & 255u));
            w4[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint4 *>(mag + (size_t)e * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
    for (uint32_t s7 = tid; s7 < 128u; s7 += nthreads) {
        const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
        uint32_t w4[4];
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) w4[i] = (((s8 >> (2u * i)) & 1u) << 15) | (((s8 >> (2u * i + 1u)) & 1u) << 31);
        *reinterpret_cast<uint4 *>(sgn + (size_t)s7 * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
}

// the eight signed fp16 weights of grid entry q of a group word, times the group's 2 s + 1
__device__ __forceinline__ half8_t decode_scaled(uint2 w, uint32_t q, const uint8_t *mag, const uint8_t *sgn) {
    const uint32_t idx = __builtin_amdgcn_ubfe(w.x, 8u * q, 8u), s7 = __builtin_amdgcn_ubfe(w.y, 7u * q, 7u);
    const uint4 m = *reinterpret_cast<const uint4 *>(mag + ((((w.y >> 28) << 8) | idx) << 4));
    const uint4 g = *reinterpret_cast<const uint4 *>(sgn + (s7 << 4));
    Half8 r;
    r.u = make_uint4(m.x ^ g.x, m.y ^ g.y, m.z ^ g.z, m.w ^ g.w);
    return r.v;
}

struct RowChunk { uint4 a, b; uint32_t d, sc; };      // four groups (32 bytes) of one packed row, the block scale over them, IQ2_XS: their four scale bytes

struct TiledArgs {
    PrefillArgs p;
    const uint8_t *experts, *shared;      // tile-major copies; same expert stride and matrix offsets as the packed layout
    float *act_f32;                       // gate/up kernel: when set, the SwiGLU activations go here as f32 [pairs][ffn] (kernels on raw rows follow)
    const int8_t *grid;                   // FMT 1 / 2: the caller's codebook; `experts` are then the row-major streams of the format
    uint64_t down_off;                    // down kernel, FMT 1 / 2: offset of the down matrix inside an expert's slot
};

// The same kernels serve IQ2_XS (FMT 1) and IQ1_M (FMT 2) matrices, read from tile-major copies of their streams (uint2 per 32 weights, d
// per 256, IQ2_XS a scale byte per 32, laid out as tile_packed_kernel writes them: a wave-wide load is 512 contiguous bytes; from the
// row-major streams, 16 rows x 32 bytes per load, the IQ2_XS down kernel took 140 us per chunk of 512 tokens). Their codebooks are too large to
// be multiplied out with every group scale, so the table holds the plain fp16 entries (8 KB / 32 KB) and the scale (per 16 weights) is
// applied to the eight weights by packed fp16 multiplies, exact: IQ2_XS entry * (2 s + 1) <= 43 * 31, IQ1_M (entry +- 1/8) * (2 s + 1)
// in eighths <= 135. The d/8 of IQ2_XS stays in the activation scale, IQ1_M has none.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// (FMT 3: IQ2_XS streams like FMT 1, decoded through a table of the codebook multiplied out with the sixteen odd scales, 128 KB: for
// kernels that have the LDS to spare, it saves the four packed multiplies per eight weights)
constexpr uint32_t kScaledXsBytes = 16u * 512u * 16u;       // [scale nibble][codebook entry]
template <int FMT> constexpr uint32_t reg_table_bytes() {
    return FMT == 0 ? kSignBytes + kScaledMagBytes : FMT == 1 ? kSignBytes + 512u * 16u : FMT == 3 ? kSignBytes + kScaledXsBytes : 2048u * 16u;
}

__device__ __forceinline__ void build_sign_table(uint8_t *sgn, uint32_t tid, uint32_t nthreads) {
    for (uint32_t s7 = tid; s7 < 128u; s7 += nthreads) {
        const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
        uint32_t w4[4];
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) w4[i] = (((s8 >> (2u * i)) & 1u) << 15) | (((s8 >> (2u * i + 1u)) & 1u) << 31);
        *reinterpret_cast<uint4 *>(sgn + (size_t)s7 * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
}
// tables of a format at `tables`: FMT 0 signs | scaled magnitudes, FMT 1 signs | fp16 codebook, FMT 2 fp16 codebook
template <int FMT>
__device__ __forceinline__ void build_reg_tables(uint8_t *tables, uint32_t tid, uint32_t nthreads, const int8_t *grid) {
    if constexpr (FMT == 0) {
        build_scaled_tables(tables + kSignBytes, tables, tid, nthreads);
    } else if constexpr (FMT == 1) {
        build_sign_table(tables, tid, nthreads);
        build_codebook_table<1>(tables + kSignBytes, tid, grid, 0u, nthreads);
    } else if constexpr (FMT == 3) {
        build_sign_table(tables, tid, nthreads);
        for (uint32_t e = tid; e < 16u * 512u; e += nthreads) {      // entries are at most 43, scales at most 31: exact in fp16
            const uint64_t ge = reinterpret_cast<const uint64_t *>(grid)[e & 511u];
            const float f = (float)(2u * (e >> 9) + 1u);
            uint32_t w4[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const _Float16 lo = (_Float16)(f * (float)(int8_t)(ge >> (16 * i))), hi = (_Float16)(f * (float)(int8_t)(ge >> (16 * i + 8)));
                w4[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
            }
            *reinterpret_cast<uint4 *>(tables + kSignBytes + (size_t)e * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
        }
    } else {
        build_codebook_table<2>(tables, tid, grid, 0u, nthreads);
    }
}
// odd integer 2 s + 1 (s < 16) as two equal fp16 halves
__device__ __forceinline__ uint32_t odd_scale_splat(uint32_t s) {
    const uint32_t h = __builtin_bit_cast(uint16_t, (_Float16)(float)(2u * s + 1u));
    return h | (h << 16);
}
// The decode in two steps, so that a kernel can have the table reads of the next groups in flight while it finishes this one:
// fetch_reg issues the LDS reads of entry q (eight columns) of a group, finish_reg turns what they returned into the eight signed,
// scaled fp16 weights. w = the group's uint2, sc = its IQ2_XS scale byte.
struct RawEntry { uint4 m, g; };
template <int FMT>
__device__ __forceinline__ RawEntry fetch_reg(uint2 w, uint32_t q, const uint8_t *tables) {
    RawEntry e;
    if constexpr (FMT == 0) {
        const uint32_t idx = __builtin_amdgcn_ubfe(w.x, 8u * q, 8u), s7 = __builtin_amdgcn_ubfe(w.y, 7u * q, 7u);
        e.m = *reinterpret_cast<const uint4 *>(tables + kSignBytes + ((((w.y >> 28) << 8) | idx) << 4));
        e.g = *reinterpret_cast<const uint4 *>(tables + (s7 << 4));
    } else if constexpr (FMT == 1) {
        const uint32_t w16 = (((q & 2u) ? w.y : w.x) >> (16u * (q & 1u))) & 0xffffu;
        e.m = *reinterpret_cast<const uint4 *>(tables + kSignBytes + ((w16 & 511u) << 4));
        e.g = *reinterpret_cast<const uint4 *>(tables + ((w16 >> 9) << 4));
    } else {
        const uint32_t idx = ((w.x >> (8u * q)) & 255u) | (((w.y >> (4u * q)) & 7u) << 8);
        e.m = *reinterpret_cast<const uint4 *>(tables + (idx << 4));
        e.g = e.m;
    }
    return e;
}
template <int FMT>
__device__ __forceinline__ half8_t finish_reg(const RawEntry &e, uint2 w, uint32_t sc, uint32_t q) {
    const uint4 m = e.m, g = e.g;
    Half8 r;
    if constexpr (FMT == 0) {
        r.u = make_uint4(m.x ^ g.x, m.y ^ g.y, m.z ^ g.z, m.w ^ g.w);
    } else if constexpr (FMT == 1) {
        const half2_t f = __builtin_bit_cast(half2_t, odd_scale_splat((sc >> (4u * (q >> 1))) & 15u));
        r.u = make_uint4(__builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.x ^ g.x) * f), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.y ^ g.y) * f),
                         __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.z ^ g.z) * f), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.w ^ g.w) * f));
    } else {
        const uint32_t fs = odd_scale_splat((w.y >> (16u + 3u * (q >> 1))) & 7u);
        const half2_t f = __builtin_bit_cast(half2_t, fs);
        const half2_t off = __builtin_bit_cast(half2_t, (fs - 0x0c000c00u) ^ (((w.y >> (4u * q + 3u)) & 1u) * 0x80008000u));
        r.u = make_uint4(__builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.x) * f + off), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.y) * f + off),
                         __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.z) * f + off), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.w) * f + off));
    }
    return r.v;
}
// both steps at once
template <int FMT>
__device__ __forceinline__ half8_t decode_reg(uint2 w, uint32_t sc, uint32_t q, const uint8_t *tables) {
    if constexpr (FMT == 0) {
        return decode_scaled(w, q, tables + kSignBytes, tables);
    } else if constexpr (FMT == 1) {
        const uint32_t w16 = (((q & 2u) ? w.y : w.x) >> (16u * (q & 1u))) & 0xffffu;
        const uint4 m = *reinterpret_cast<const uint4 *>(tables + kSignBytes + ((w16 & 511u) << 4));
        const uint4 g = *reinterpret_cast<const uint4 *>(tables + ((w16 >> 9) << 4));
        const half2_t f = __builtin_bit_cast(half2_t, odd_scale_splat((sc >> (4u * (q >> 1))) & 15u));
        Half8 r;
        r.u = make_uint4(__builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.x ^ g.x) * f), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.y ^ g.y) * f),
                         __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.z ^ g.z) * f), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.w ^ g.w) * f));
        return r.v;
    } else if constexpr (FMT == 3) {
        const uint32_t w16 = (((q & 2u) ? w.y : w.x) >> (16u * (q & 1u))) & 0xffffu;
        const uint32_t nib = (sc >> (4u * (q >> 1))) & 15u;
        const uint4 m = *reinterpret_cast<const uint4 *>(tables + kSignBytes + (((nib << 9) | (w16 & 511u)) << 4));
        const uint4 g = *reinterpret_cast<const uint4 *>(tables + ((w16 >> 9) << 4));
        Half8 r;
        r.u = make_uint4(m.x ^ g.x, m.y ^ g.y, m.z ^ g.z, m.w ^ g.w);
        return r.v;
    } else {
        const uint32_t idx = ((w.x >> (8u * q)) & 255u) | (((w.y >> (4u * q)) & 7u) << 8);
        const uint4 m = *reinterpret_cast<const uint4 *>(tables + (idx << 4));
        const uint32_t fs = odd_scale_splat((w.y >> (16u + 3u * (q >> 1))) & 7u);
        const half2_t f = __builtin_bit_cast(half2_t, fs);
        // (2 s + 1) / 8 with the sign of the offset: three exponent steps down (2 s + 1 >= 1 is a normal number), sign bit by xor
        const half2_t off = __builtin_bit_cast(half2_t, (fs - 0x0c000c00u) ^ (((w.y >> (4u * q + 3u)) & 1u) * 0x80008000u));
        Half8 r;
        r.u = make_uint4(__builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.x) * f + off), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.y) * f + off),
                         __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.z) * f + off), __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, m.w) * f + off));
        return r.v;
    }
}

// gate/up + SwiGLU. Wave = (K quarter kc, column half rh): for the unit of 32 FFN columns j it computes the gate row and the
// up row of column 32 j + 16 rh + r against its quarter of the hidden dimension; the quarters meet in LDS (double-buffered:
// one barrier per unit).
// Work items are parts of tiles (128 of the FFN columns, with an activation exponent of their own) so that the last round of
// the persistent workgroups is short (with half tiles as items a chunk of 544 tiles gave four items to some workgroups and five
// to others); a workgroup takes a contiguous range of items and keeps its A operands when consecutive ones share a tile.
// Items item_begin .. item_end - 1 (item = tile * parts + part) of the tile list in ta.p; `tables` built by the caller (a barrier of this
// function comes before their first use); lds: [16][128 + 4] f32 activations, then the partial sums [unit parity][K quarter][pair][gate
// 0..31 | up 0..31, padded to 68] f32; tok_scale / tok_of: 16 entries each.
constexpr size_t kNarrowLds = ((size_t)kTile * (32u * kItemUnits + 4u) + (size_t)2u * 4u * kTile * 68u) * sizeof(float);
template <int NKC, int FMT>          // hidden = 512 * NKC; FMT 0: tile-major packed IQ2_XXS, 1 / 2: row-major IQ2_XS / IQ1_M streams
__device__ __forceinline__ void gateup_narrow_items(const TiledArgs &ta, uint32_t item_begin, uint32_t item_end, const uint8_t *tables, uint8_t *lds,
                                                    float *tok_scale, uint32_t *tok_of) {
    const PrefillArgs &a = ta.p;
    constexpr uint32_t H = 512u * NKC, HG = H / 32u, HB = H / 256u, GQ = HG / 4u, NC = H / 128u;   // GQ: groups per K quarter = 4 NKC
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), kc = wave & 3u, rh = wave >> 2;
    const uint32_t F = a.ffn, FG = F / 32u, P = a.ntok * a.top_k;
    constexpr uint32_t FGH = kItemUnits, AROW = 32u * kItemUnits + 4u;
    float *acts = reinterpret_cast<float *>(lds);
    float (*part)[4][kTile][68] = reinterpret_cast<float (*)[4][kTile][68]>(acts + kTile * AROW);
    const uint32_t U = a.n_unique[0];
    const uint64_t qs_bytes = (uint64_t)F * HG * 8u, sc_off = qs_bytes + (uint64_t)F * HB * 2u, gate_bytes = sc_off + (FMT == 1 ? (uint64_t)F * HG : 0u);
    const uint32_t parts = FG / FGH;
    Half8 xa[GQ], xb[GQ];
    uint32_t have_tile = 0xffffffffu;
    // An item's tile entry, its expert's address and its first weight chunks are three dependent round trips: those of the next item are
    // requested while this one is multiplied (the last chunk step of an item fetches the next item's first chunks instead of its own again).
    struct ItemInfo { uint32_t p0, n; const uint8_t *ex; };
    auto info_of = [&](uint32_t item) {
        const uint32_t tile = item / parts;
        const uint32_t u = a.tile_group[tile];
        return ItemInfo{a.tile_pair0[tile], a.tile_n[tile], u == U ? ta.shared : ta.experts + (uint64_t)a.uid[u] * a.stride};
    };
    auto load_chunk = [&](const uint8_t *mat, uint32_t j, uint32_t c) {
        const uint32_t rtile = 2u * j + rh, chunk = kc * NKC + c;
        const uint64_t at = ((uint64_t)rtile * NC + chunk) * 16u + r;
        const uint4 *qp = reinterpret_cast<const uint4 *>(mat + at * 32u);
        const uint16_t *dp = reinterpret_cast<const uint16_t *>(mat + qs_bytes) + ((uint64_t)rtile * HB + chunk / 2u) * 16u + r;
        return RowChunk{qp[0], qp[1], *dp, FMT == 1 ? reinterpret_cast<const uint32_t *>(mat + sc_off)[at] : 0u};
    };
    if (item_begin >= item_end) return;
    ItemInfo cur = info_of(item_begin);
    RowChunk cg = load_chunk(cur.ex, (item_begin % parts) * FGH, 0u), cu = load_chunk(cur.ex + gate_bytes, (item_begin % parts) * FGH, 0u);
    for (uint32_t item = item_begin; item < item_end; ++item) {
        const uint32_t tile = item / parts, ipart = item % parts, j0 = ipart * FGH;
        const uint32_t p0 = cur.p0, n = cur.n;
        const uint8_t *ex = cur.ex;
        const uint32_t next_item = item + 1u < item_end ? item + 1u : item;
        const ItemInfo nxt = info_of(next_item);
        const uint32_t next_j0 = (next_item % parts) * FGH;
        __syncthreads();                                   // the previous item's readers are done with acts / tok_of; tables are built
        if (tile != have_tile) {
            have_tile = tile;
            if (tid < kTile) {
                const uint32_t p = p0 + tid, tok = tid < n ? (p < P ? a.pair_token[p] : p - P) : 0u;
                tok_of[tid] = tok;
                tok_scale[tid] = tid < n ? (FMT == 2 ? 1.0f : 0.125f) * exp2i(a.xexp[tok]) : 0.0f;
            }
            __syncthreads();
            // this lane's A operands for the whole tile: token of pair r, columns 8 q .. 8 q + 7 of each group of the wave's quarter
            const uint64_t base = (uint64_t)tok_of[r] * H + 32u * (kc * GQ) + 8u * q;
            const bool live = r < n;
#pragma unroll
            for (uint32_t g = 0; g < GQ; ++g) {
                xa[g].u = make_uint4(0u, 0u, 0u, 0u);
                xb[g].u = xa[g].u;
                if (live) {
                    xa[g].u = *reinterpret_cast<const uint4 *>(a.xh + base + 32u * g);
                    xb[g].u = *reinterpret_cast<const uint4 *>(a.xl + base + 32u * g);
                }
            }
        }
        const uint8_t *gmat = ex;
#pragma unroll 1
        for (uint32_t j = j0; j < j0 + FGH; ++j) {
            float4_t totg = {0.0f, 0.0f, 0.0f, 0.0f}, totu = totg;
#pragma unroll
            for (uint32_t c = 0; c < (uint32_t)NKC; ++c) {
                // the chunk after this one (same unit, the first of the next unit, or the first of the next item) is in flight
                const bool to_next_item = c + 1u == (uint32_t)NKC && j + 1u == j0 + FGH;
                const uint32_t nj = c + 1u < (uint32_t)NKC ? j : (to_next_item ? next_j0 : j + 1u), nc = c + 1u < (uint32_t)NKC ? c + 1u : 0u;
                const uint8_t *ngm = to_next_item ? nxt.ex : gmat;
                const RowChunk ng = load_chunk(ngm, nj, nc), nu = load_chunk(ngm + gate_bytes, nj, nc);
                __builtin_amdgcn_sched_barrier(0);         // keeps the loads ahead of the chunk's arithmetic
                const uint2 wg4[4] = {make_uint2(cg.a.x, cg.a.y), make_uint2(cg.a.z, cg.a.w), make_uint2(cg.b.x, cg.b.y), make_uint2(cg.b.z, cg.b.w)};
                const uint2 wu4[4] = {make_uint2(cu.a.x, cu.a.y), make_uint2(cu.a.z, cu.a.w), make_uint2(cu.b.x, cu.b.y), make_uint2(cu.b.z, cu.b.w)};
                // the four groups of the chunk share the block scale d: their products add up in the matrix units, activations
                // hi and lo in accumulators of their own
                float4_t gh = {0.0f, 0.0f, 0.0f, 0.0f}, gl = gh, uh = gh, ul = gh;
                // the table reads run two groups ahead of the arithmetic: a wave that waits for every read before it issues the next
                // spends most of its time on LDS round trips (two waves per SIMD do not hide them)
                RawEntry rg0 = fetch_reg<FMT>(wg4[0], q, tables), ru0 = fetch_reg<FMT>(wu4[0], q, tables);
                RawEntry rg1 = fetch_reg<FMT>(wg4[1], q, tables), ru1 = fetch_reg<FMT>(wu4[1], q, tables);
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) {
                    const uint32_t g = 4u * c + k;
                    __builtin_amdgcn_sched_barrier(0);
                    const half8_t bg = finish_reg<FMT>(k & 1u ? rg1 : rg0, wg4[k], cg.sc >> (8u * k), q), bu = finish_reg<FMT>(k & 1u ? ru1 : ru0, wu4[k], cu.sc >> (8u * k), q);
                    if (k + 2u < 4u) {
                        if (k & 1u) { rg1 = fetch_reg<FMT>(wg4[k + 2u], q, tables); ru1 = fetch_reg<FMT>(wu4[k + 2u], q, tables); }
                        else { rg0 = fetch_reg<FMT>(wg4[k + 2u], q, tables); ru0 = fetch_reg<FMT>(wu4[k + 2u], q, tables); }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    gh = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[g].v, bg, gh, 0, 0, 0);
                    gl = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[g].v, bg, gl, 0, 0, 0);
                    uh = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[g].v, bu, uh, 0, 0, 0);
                    ul = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[g].v, bu, ul, 0, 0, 0);
                }
                const float dg = scale_to_f32(cg.d), du = scale_to_f32(cu.d);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    totg[t] = fmaf(fmaf(gl[t], 4.8828125e-4f, gh[t]), dg, totg[t]);
                    totu[t] = fmaf(fmaf(ul[t], 4.8828125e-4f, uh[t]), du, totu[t]);
                }
                cg = ng;
                cu = nu;
            }
            float (*pt)[kTile][68] = part[j & 1u];
#pragma unroll
            for (uint32_t t = 0; t < 4u; ++t) {
                pt[kc][4u * q + t][16u * rh + r] = totg[t];
                pt[kc][4u * q + t][32u + 16u * rh + r] = totu[t];
            }
            __syncthreads();
            {   // (pair i, column c) per thread: the four quarters, the token's scale, SwiGLU
                const uint32_t i = tid >> 5, c = tid & 31u;
                const float gsum = ((pt[0][i][c] + pt[1][i][c]) + (pt[2][i][c] + pt[3][i][c])) * tok_scale[i];
                const float usum = ((pt[0][i][32u + c] + pt[1][i][32u + c]) + (pt[2][i][32u + c] + pt[3][i][32u + c])) * tok_scale[i];
                acts[i * AROW + 32u * (j - j0) + c] = (gsum / (1.0f + expf(-gsum))) * usum;
            }
        }
        __syncthreads();
        // one exponent per pair and part, then the fp16 halves: wave w takes pairs 2 w and 2 w + 1
        const uint32_t c0 = 32u * j0, c1 = c0 + 32u * FGH;
#pragma unroll
        for (uint32_t h = 0; h < 2u; ++h) {
            const uint32_t i = 2u * wave + h;
            if (i >= n) continue;                          // wave-uniform
            if (ta.act_f32) {
                for (uint32_t c = c0 + lane; c < c1; c += 64u) ta.act_f32[(uint64_t)(p0 + i) * F + c] = acts[i * AROW + c - c0];
                continue;
            }
            float amax = 0.0f;
            for (uint32_t c = c0 + lane; c < c1; c += 64u) amax = fmaxf(amax, fabsf(acts[i * AROW + c - c0]));
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const int e = prescale_exp(amax);
            const float inv = exp2i(-e);
            const uint64_t pr = p0 + i;
            for (uint32_t c = c0 + lane; c < c1; c += 64u) split_hi_lo(acts[i * AROW + c - c0], inv, a.act_h + pr * F + c, a.act_l + pr * F + c);
            if (lane == 0u) a.act_exp[kExpPerPair * pr + ipart] = e;
        }
        cur = nxt;
    }
}

// the kernel of hidden 512: all items of the list in ta.p
template <int NKC, int FMT>
__global__ __launch_bounds__(kRegWaves * 64) void prefill_gateup_reg_kernel(TiledArgs ta) {
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];
    __shared__ __attribute__((aligned(16))) uint8_t tables[reg_table_bytes<FMT>()];      // static: table reads take immediate offsets
    __shared__ float tok_scale[kTile];
    __shared__ uint32_t tok_of[kTile];
    build_reg_tables<FMT>(tables, threadIdx.x, kRegWaves * 64u, ta.grid);
    const uint32_t items = (ta.p.ffn / 32u / kItemUnits) * ta.p.n_tiles[0];
    gateup_narrow_items<NKC, FMT>(ta, (uint32_t)(((uint64_t)blockIdx.x * items) / gridDim.x), (uint32_t)(((uint64_t)(blockIdx.x + 1u) * items) / gridDim.x), tables, dyn,
                                  tok_scale, tok_of);
}

// The same gate/up + SwiGLU on the wide tiles (17 .. 32 pairs, list 1 of build_tiles_kernel): a wave owns an eighth of the hidden
// dimension and keeps the activations of two sets of 16 pairs for it in registers (the same 128 registers as a quarter for one set); for
// every unit of 32 FFN columns it decodes both row halves of its eighth and multiplies each decoded operand with both sets, so an expert
// with many pairs in the chunk is decoded once per 32 of them. The eight partial sums per (pair, column) meet in LDS, single-buffered:
// two barriers per unit. (On tiles of 16 or fewer pairs this layout was measured a quarter slower than the kernel above: they stay there.)
// lds: [32][128 + 4] f32 activations, then the partial sums [8 K eighths][32 pairs][gate 0..31 | up 0..31, padded to 68] f32; tok_scale /
// tok_of: 32 entries each; the rest as gateup_narrow_items.
constexpr size_t kWideLds = ((size_t)kWideTile * (32u * kItemUnits + 4u) + (size_t)8u * kWideTile * 68u) * sizeof(float);
template <int NKC, int FMT>          // hidden = 512 * NKC, NKC even
__device__ __forceinline__ void gateup_wide_items(const TiledArgs &ta, uint32_t item_begin, uint32_t item_end, const uint8_t *tables, uint8_t *lds,
                                                  float *tok_scale, uint32_t *tok_of) {
    static_assert(NKC % 2 == 0 && kRegWaves == 8, "a wave takes NKC / 2 chunks of 128 columns");
    const PrefillArgs &a = ta.p;
    constexpr uint32_t H = 512u * NKC, HG = H / 32u, HB = H / 256u, GE = HG / 8u, NC = H / 128u, CW = NKC / 2u;   // GE: groups per K eighth = 2 NKC; CW: chunks per wave
    constexpr uint32_t FGH = kItemUnits, AROW = 32u * kItemUnits + 4u;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t kc = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t F = a.ffn, FG = F / 32u, P = a.ntok * a.top_k;
    float *acts = reinterpret_cast<float *>(lds);
    float (*part)[kWideTile][68] = reinterpret_cast<float (*)[kWideTile][68]>(acts + kWideTile * AROW);
    const uint32_t U = a.n_unique[0];
    const uint64_t qs_bytes = (uint64_t)F * HG * 8u, sc_off = qs_bytes + (uint64_t)F * HB * 2u, gate_bytes = sc_off + (FMT == 1 ? (uint64_t)F * HG : 0u);
    const uint32_t parts = FG / FGH;
    Half8 xa[2][GE], xb[2][GE];
    uint32_t have_tile = 0xffffffffu;
    for (uint32_t item = item_begin; item < item_end; ++item) {
        const uint32_t tile = item / parts, ipart = item % parts, j0 = ipart * FGH;
        const uint32_t u = a.tile_group[tile], p0 = a.tile_pair0[tile], n = a.tile_n[tile];
        const uint8_t *ex = u == U ? ta.shared : ta.experts + (uint64_t)a.uid[u] * a.stride;
        __syncthreads();                                   // the previous item's readers are done with acts / tok_of; tables are built
        if (tile != have_tile) {
            have_tile = tile;
            if (tid < kWideTile) {
                const uint32_t p = p0 + tid, tok = tid < n ? (p < P ? a.pair_token[p] : p - P) : 0u;
                tok_of[tid] = tok;
                tok_scale[tid] = tid < n ? (FMT == 2 ? 1.0f : 0.125f) * exp2i(a.xexp[tok]) : 0.0f;
            }
            __syncthreads();
#pragma unroll
            for (uint32_t s2 = 0; s2 < 2u; ++s2) {
                const uint64_t base = (uint64_t)tok_of[16u * s2 + r] * H + 32u * (kc * GE) + 8u * q;
                const bool live = 16u * s2 + r < n;
#pragma unroll
                for (uint32_t g = 0; g < GE; ++g) {
                    xa[s2][g].u = make_uint4(0u, 0u, 0u, 0u);
                    xb[s2][g].u = xa[s2][g].u;
                    if (live) {
                        xa[s2][g].u = *reinterpret_cast<const uint4 *>(a.xh + base + 32u * g);
                        xb[s2][g].u = *reinterpret_cast<const uint4 *>(a.xl + base + 32u * g);
                    }
                }
            }
            // The low halves are stored times 2^11; here they go back to their own scale (exact: the largest |x| of a token sits in
            // [2^13, 2^14), so a low half below the fp16 normal range belongs to an element 2^-16 of that), and a product's high and low
            // parts add up in one accumulator.
#pragma unroll
            for (uint32_t s2 = 0; s2 < 2u; ++s2)
#pragma unroll
                for (uint32_t g = 0; g < GE; ++g) xb[s2][g].v = xb[s2][g].v * (_Float16)4.8828125e-4f;
        }
        // half step hs of the item: unit j0 + hs / 2, row half hs % 2; chunks c = 0 .. CW - 1 of the wave's eighth inside it
        constexpr uint32_t kHalfSteps = FGH * 2u;
        auto load_chunk = [&](const uint8_t *mat, uint32_t hs, uint32_t c) {
            const uint32_t rtile = 2u * j0 + hs, chunk = kc * CW + c;      // (2 (j0 + hs / 2) + hs % 2)
            const uint64_t at = ((uint64_t)rtile * NC + chunk) * 16u + r;
            const uint4 *qp = reinterpret_cast<const uint4 *>(mat + at * 32u);
            const uint16_t *dp = reinterpret_cast<const uint16_t *>(mat + qs_bytes) + ((uint64_t)rtile * HB + chunk / 2u) * 16u + r;
            return RowChunk{qp[0], qp[1], *dp, FMT == 1 ? reinterpret_cast<const uint32_t *>(mat + sc_off)[at] : 0u};
        };
        const uint8_t *gmat = ex, *umat = ex + gate_bytes;
        RowChunk cg = load_chunk(gmat, 0u, 0u), cu = load_chunk(umat, 0u, 0u);
#pragma unroll 1
        for (uint32_t hs = 0; hs < kHalfSteps; ++hs) {
            const uint32_t rh = hs & 1u, j = j0 + (hs >> 1);
            float4_t totg[2], totu[2];
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) { totg[s2] = float4_t{0.0f, 0.0f, 0.0f, 0.0f}; totu[s2] = totg[s2]; }
#pragma unroll
            for (uint32_t c = 0; c < CW; ++c) {
                // the chunk after this one (same half step, or the first of the next; the last one reloads itself) is in flight
                const uint32_t nh = c + 1u < CW ? hs : (hs + 1u < kHalfSteps ? hs + 1u : hs), nc = c + 1u < CW ? c + 1u : 0u;
                const RowChunk ng = load_chunk(gmat, nh, nc), nu = load_chunk(umat, nh, nc);
                __builtin_amdgcn_sched_barrier(0);         // keeps the loads ahead of the chunk's arithmetic
                const uint2 wg4[4] = {make_uint2(cg.a.x, cg.a.y), make_uint2(cg.a.z, cg.a.w), make_uint2(cg.b.x, cg.b.y), make_uint2(cg.b.z, cg.b.w)};
                const uint2 wu4[4] = {make_uint2(cu.a.x, cu.a.y), make_uint2(cu.a.z, cu.a.w), make_uint2(cu.b.x, cu.b.y), make_uint2(cu.b.z, cu.b.w)};
                float4_t ga[2], ua[2];
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2) { ga[s2] = float4_t{0.0f, 0.0f, 0.0f, 0.0f}; ua[s2] = ga[s2]; }
                RawEntry rg0 = fetch_reg<FMT>(wg4[0], q, tables), ru0 = fetch_reg<FMT>(wu4[0], q, tables);
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) {
                    const uint32_t g = 4u * c + k;
                    __builtin_amdgcn_sched_barrier(0);
                    const half8_t bg = finish_reg<FMT>(rg0, wg4[k], cg.sc >> (8u * k), q), bu = finish_reg<FMT>(ru0, wu4[k], cu.sc >> (8u * k), q);
                    if (k + 1u < 4u) { rg0 = fetch_reg<FMT>(wg4[k + 1u], q, tables); ru0 = fetch_reg<FMT>(wu4[k + 1u], q, tables); }
                    __builtin_amdgcn_sched_barrier(0);
                    ga[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[0][g].v, bg, ga[0], 0, 0, 0);
                    ua[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[0][g].v, bu, ua[0], 0, 0, 0);
                    ga[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[1][g].v, bg, ga[1], 0, 0, 0);
                    ua[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[1][g].v, bu, ua[1], 0, 0, 0);
                    ga[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[0][g].v, bg, ga[0], 0, 0, 0);
                    ua[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[0][g].v, bu, ua[0], 0, 0, 0);
                    ga[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[1][g].v, bg, ga[1], 0, 0, 0);
                    ua[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[1][g].v, bu, ua[1], 0, 0, 0);
                }
                const float dg = scale_to_f32(cg.d), du = scale_to_f32(cu.d);
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        totg[s2][t] = fmaf(ga[s2][t], dg, totg[s2][t]);
                        totu[s2][t] = fmaf(ua[s2][t], du, totu[s2][t]);
                    }
                cg = ng;
                cu = nu;
            }
            // this row half of the unit is complete for the wave's eighth
#pragma unroll
            for (uint32_t s2 = 0; s2 < 2u; ++s2)
#pragma unroll
                for (uint32_t t = 0; t < 4u; ++t) {
                    part[kc][16u * s2 + 4u * q + t][16u * rh + r] = totg[s2][t];
                    part[kc][16u * s2 + 4u * q + t][32u + 16u * rh + r] = totu[s2][t];
                }
            if (rh == 0u) continue;
            __syncthreads();
            for (uint32_t i = tid >> 5; i < kWideTile; i += 16u) {      // (pair i, column cc) per thread: the eight eighths, the token's scale, SwiGLU
                const uint32_t cc = tid & 31u;
                float gs[8], us[8];
#pragma unroll
                for (int e8 = 0; e8 < 8; ++e8) { gs[e8] = part[e8][i][cc]; us[e8] = part[e8][i][32u + cc]; }
                const float gsum = (((gs[0] + gs[1]) + (gs[2] + gs[3])) + ((gs[4] + gs[5]) + (gs[6] + gs[7]))) * tok_scale[i];
                const float usum = (((us[0] + us[1]) + (us[2] + us[3])) + ((us[4] + us[5]) + (us[6] + us[7]))) * tok_scale[i];
                acts[i * AROW + 32u * (j - j0) + cc] = (gsum / (1.0f + expf(-gsum))) * usum;
            }
            __syncthreads();                               // the partial sums may be overwritten
        }
        // one exponent per pair and part, then the fp16 halves: wave w takes pairs 4 w .. 4 w + 3
        const uint32_t c0 = 32u * j0, c1 = c0 + 32u * FGH;
#pragma unroll
        for (uint32_t h = 0; h < 4u; ++h) {
            const uint32_t i = 4u * kc + h;
            if (i >= n) continue;                          // wave-uniform
            if (ta.act_f32) {
                for (uint32_t c = c0 + lane; c < c1; c += 64u) ta.act_f32[(uint64_t)(p0 + i) * F + c] = acts[i * AROW + c - c0];
                continue;
            }
            float amax = 0.0f;
            for (uint32_t c = c0 + lane; c < c1; c += 64u) amax = fmaxf(amax, fabsf(acts[i * AROW + c - c0]));
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const int e = prescale_exp(amax);
            const float inv = exp2i(-e);
            const uint64_t pr = p0 + i;
            for (uint32_t c = c0 + lane; c < c1; c += 64u) split_hi_lo(acts[i * AROW + c - c0], inv, a.act_h + pr * F + c, a.act_l + pr * F + c);
            if (lane == 0u) a.act_exp[kExpPerPair * pr + ipart] = e;
        }
    }
}

// Gate/up of a chunk in one launch: the wide tiles (list 1, at ta.p's tile arrays + list_stride) and the narrow ones (list 2). The
// persistent workgroups cut one line of work into equal pieces: first the wide items at 3 units each, then the narrow ones at 2 (a wide
// item was measured at 1.4 narrow ones); a workgroup runs the items that start inside its piece, so every compute unit is busy whatever
// the mix (as two launches the wide tiles of a chunk with few of them left half of the device idle: 171 against 157 us).
template <int NKC, int FMT>
__global__ __launch_bounds__(kRegWaves * 64) void prefill_gateup_mixed_kernel(TiledArgs ta, uint32_t list_stride) {
    extern __shared__ __attribute__((aligned(16))) uint8_t dyn[];          // kWideLds
    __shared__ __attribute__((aligned(16))) uint8_t tables[reg_table_bytes<FMT>()];      // static: table reads take immediate offsets
    __shared__ float tok_scale[kWideTile];
    __shared__ uint32_t tok_of[kWideTile];
    build_reg_tables<FMT>(tables, threadIdx.x, kRegWaves * 64u, ta.grid);
    const uint32_t parts = ta.p.ffn / 32u / kItemUnits, n_wide = parts * ta.p.n_tiles[1], n_narrow = parts * ta.p.n_tiles[2];
    const uint64_t line = 3ull * n_wide + 2ull * n_narrow;
    const uint64_t lo = (uint64_t)blockIdx.x * line / gridDim.x, hi = (uint64_t)(blockIdx.x + 1u) * line / gridDim.x;
    // items whose start (3 i, or 3 n_wide + 2 j) lies in [lo, hi)
    const auto first_at = [](uint64_t x, uint64_t base, uint64_t unit, uint32_t n) { const uint64_t i = x <= base ? 0u : (x - base + unit - 1u) / unit; return (uint32_t)(i < n ? i : n); };
    const uint32_t w0 = first_at(lo, 0u, 3u, n_wide), w1 = first_at(hi, 0u, 3u, n_wide);
    const uint32_t m0 = first_at(lo, 3ull * n_wide, 2u, n_narrow), m1 = first_at(hi, 3ull * n_wide, 2u, n_narrow);
    TiledArgs tl = ta;
    const auto use_list = [&](uint32_t l) {
        tl.p.tile_group = ta.p.tile_group + l * list_stride;
        tl.p.tile_pair0 = ta.p.tile_pair0 + l * list_stride;
        tl.p.tile_n = ta.p.tile_n + l * list_stride;
    };
    use_list(1u);
    gateup_wide_items<NKC, FMT>(tl, w0, w1, tables, dyn, tok_scale, tok_of);
    use_list(2u);
    gateup_narrow_items<NKC, FMT>(tl, m0, m1, tables, dyn, tok_scale, tok_of);
}

// down. Wave w computes rows 128 b + 16 w + r for b = 0, 1, ... against all ffn columns of the tile; no reduction across waves.
template <int NFG, int FMT>          // ffn = 32 * NFG, NFG <= 16; FMT as in the gate/up kernel
__global__ __launch_bounds__(kRegWaves * 64) void prefill_down_reg_kernel(TiledArgs ta) {
    const PrefillArgs &a = ta.p;
    constexpr uint32_t F = 32u * NFG, FB = F / 256u, NCK = NFG / 4u;
    __shared__ __attribute__((aligned(16))) uint8_t tables[reg_table_bytes<FMT>()];      // static: table reads take immediate offsets
    __shared__ __attribute__((aligned(16))) float pair_scale[kExpPerPair][kTile];      // per 128-column chunk of the activations
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t H = a.hidden, P = a.ntok * a.top_k;
    build_reg_tables<FMT>(tables, tid, kRegWaves * 64u, ta.grid);
    const uint32_t T = a.n_tiles[0], U = a.n_unique[0];
    const uint64_t down_off = FMT == 0 ? 2u * ((uint64_t)F * (H / 32u) * 8u + (uint64_t)F * (H / 256u) * 2u) : ta.down_off, qs_bytes = (uint64_t)H * NFG * 8u;
    const uint64_t sc_off = qs_bytes + (uint64_t)H * FB * 2u;
    constexpr uint32_t kRowsPerPass = 16u * kRegWaves;

    // Work items are quarter tiles (the row passes of a tile cut in four) so that the last round of the persistent workgroups is
    // short; a workgroup takes a contiguous range of items and keeps the activations when consecutive ones share a tile.
    const uint32_t n_pass_tile = H / kRowsPerPass, parts = n_pass_tile % 4u == 0u ? 4u : n_pass_tile % 2u == 0u ? 2u : 1u, n_pass = n_pass_tile / parts;
    const uint32_t items = T * parts;
    const uint32_t item_begin = (uint32_t)(((uint64_t)blockIdx.x * items) / gridDim.x), item_end = (uint32_t)(((uint64_t)(blockIdx.x + 1u) * items) / gridDim.x);
    Half8 xa[NFG], xb[NFG];
    uint32_t have_tile = 0xffffffffu;
    for (uint32_t item = item_begin; item < item_end; ++item) {
        const uint32_t tile = item / parts, pass0 = (item % parts) * n_pass;
        const uint32_t u = a.tile_group[tile], p0 = a.tile_pair0[tile], n = a.tile_n[tile];
        const uint8_t *dn = (u == U ? ta.shared : ta.experts + (uint64_t)a.uid[u] * a.stride) + down_off;
        if (tile != have_tile) {
            have_tile = tile;
            __syncthreads();
            if (tid < kExpPerPair * kTile && (tid & 3u) < NCK) pair_scale[tid & 3u][tid >> 2] = (tid >> 2) < n ? (FMT == 2 ? 1.0f : 0.125f) * exp2i(a.act_exp[kExpPerPair * p0 + tid]) : 0.0f;
            __syncthreads();
            const uint64_t base = (uint64_t)(p0 + r) * F + 8u * q;
            const bool live = r < n;
#pragma unroll
            for (uint32_t g = 0; g < (uint32_t)NFG; ++g) {
                xa[g].u = make_uint4(0u, 0u, 0u, 0u);
                xb[g].u = xa[g].u;
                if (live) {
                    xa[g].u = *reinterpret_cast<const uint4 *>(a.act_h + base + 32u * g);
                    xb[g].u = *reinterpret_cast<const uint4 *>(a.act_l + base + 32u * g);
                }
            }
        }
        auto load_chunk = [&](uint32_t b, uint32_t c) {
            const uint32_t rtile = kRegWaves * (pass0 + b) + wave;
            const uint64_t at = ((uint64_t)rtile * NCK + c) * 16u + r;
            const uint4 *qp = reinterpret_cast<const uint4 *>(dn + at * 32u);
            const uint16_t *dp = reinterpret_cast<const uint16_t *>(dn + qs_bytes) + ((uint64_t)rtile * FB + c / 2u) * 16u + r;
            return RowChunk{qp[0], qp[1], *dp, FMT == 1 || FMT == 3 ? reinterpret_cast<const uint32_t *>(dn + sc_off)[at] : 0u};
        };
        // One buffer per chunk of a pass, reloaded with the same chunk of the next pass as soon as it has been decoded: every load
        // has a whole pass of work to arrive.
        RowChunk cw[NCK];
#pragma unroll
        for (uint32_t c = 0; c < NCK; ++c) cw[c] = load_chunk(0u, c);
#pragma unroll 1
        for (uint32_t b = 0; b < n_pass; ++b) {
            float4_t tot = {0.0f, 0.0f, 0.0f, 0.0f};
            const uint32_t nb = b + 1u < n_pass ? b + 1u : b;          // the last pass reloads itself: no branch around the loads
#pragma unroll
            for (uint32_t c = 0; c < NCK; ++c) {
                const uint2 w4[4] = {make_uint2(cw[c].a.x, cw[c].a.y), make_uint2(cw[c].a.z, cw[c].a.w), make_uint2(cw[c].b.x, cw[c].b.y), make_uint2(cw[c].b.z, cw[c].b.w)};
                const float d = scale_to_f32(cw[c].d);
                const uint32_t sc4 = cw[c].sc;
                cw[c] = load_chunk(nb, c);
                __builtin_amdgcn_sched_barrier(0);         // keeps the loads here: the scheduler otherwise sinks them to the end of the pass
                float4_t hi = {0.0f, 0.0f, 0.0f, 0.0f}, lo = hi;
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) {
                    const uint32_t g = 4u * c + k;
                    const half8_t bw = decode_reg<FMT>(w4[k], sc4 >> (8u * k), q, tables);
                    hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[g].v, bw, hi, 0, 0, 0);
                    lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[g].v, bw, lo, 0, 0, 0);
                }
                const float4_t ps = *reinterpret_cast<const float4_t *>(&pair_scale[c][4u * q]);
#pragma unroll
                for (int t = 0; t < 4; ++t) tot[t] = fmaf(fmaf(lo[t], 4.8828125e-4f, hi[t]) * d, ps[t], tot[t]);
            }
            const uint32_t row = kRowsPerPass * (pass0 + b) + 16u * wave + r;
#pragma unroll
            for (uint32_t t = 0; t < 4u; ++t) {
                const uint32_t i = 4u * q + t, p = p0 + i;
                if (i < n) (p < P ? a.tmp + (uint64_t)p * H : a.sh_tmp + (uint64_t)(p - P) * H)[row] = tot[t];
            }
        }
    }
}

// ---------------------------------------------------------------- IQ3_S down projection on tiles (mixed layouts)

// Tile-major IQ3_S (built once at upload from the raw 110-byte blocks): per group of 32 weights four 32-bit words, one per eight
// weights l: bits 0-8 the first grid index, 9-17 the second (each with its ninth bit from qh), 18-25 the eight sign bits, 26-29 the
// group's scale nibble. A row's chunk of four groups is stored as [l][group] so that lane (r, l) reads its own four words as one
// 16-byte load, and the chunks of 16 consecutive rows lie next to each other (a wave-wide load is 1024 contiguous bytes):
//   chunk (row, c)  at ((row / 16 * (K / 128) + c) * 16 + row % 16) * 64,   lane l adds 16 l
//   scale (row, b)  at qs_bytes + ((row / 16 * (K / 256) + b) * 16 + row % 16) * 2
__global__ void tile_iq3s_kernel(const uint8_t *raw, uint64_t raw_stride, uint32_t nrows, uint32_t K, uint8_t *tiled, uint64_t tiled_stride) {
    const uint32_t NG = K / 32u, NC = K / 128u, NB = K / 256u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)nrows * NG) return;
    const uint32_t row = (uint32_t)(gid / NG), g = (uint32_t)(gid % NG), sub = g & 7u;
    const uint8_t *bp = raw + (uint64_t)blockIdx.y * raw_stride + ((uint64_t)row * NB + (g >> 3)) * 110u;
    uint8_t *dst = tiled + (uint64_t)blockIdx.y * tiled_stride;
    const uint32_t nib = ((uint32_t)bp[106u + (sub >> 1)] >> (4u * (sub & 1u))) & 15u, qh = bp[66u + sub];
    uint32_t *out = reinterpret_cast<uint32_t *>(dst + (((uint64_t)(row / 16u) * NC + (g >> 2)) * 16u + row % 16u) * 64u);
    for (uint32_t l = 0; l < 4u; ++l) {
        const uint32_t ia = (uint32_t)bp[2u + 8u * sub + 2u * l] | ((qh << (8u - 2u * l)) & 256u);
        const uint32_t ib = (uint32_t)bp[3u + 8u * sub + 2u * l] | ((qh << (7u - 2u * l)) & 256u);
        out[4u * l + (g & 3u)] = ia | (ib << 9) | ((uint32_t)bp[74u + 4u * sub + l] << 18) | (nib << 26);
    }
    if (sub == 0u)
        reinterpret_cast<uint16_t *>(dst + (uint64_t)nrows * NG * 16u)[((uint64_t)(row / 16u) * NB + (g >> 3)) * 16u + row % 16u] = (uint16_t)ld_u16(bp);
}

hipError_t launch_tile_iq3s(const void *raw, uint64_t raw_stride, uint32_t count, uint32_t nrows, uint32_t K, void *tiled, uint64_t tiled_stride, hipStream_t s) {
    if (!nrows || nrows % 16u || !K || K % 256u || !count || count > 65535u) return hipErrorInvalidValue;
    const uint64_t total = (uint64_t)nrows * (K / 32u);
    REDHIP_LAUNCH(tile_iq3s_kernel, dim3((uint32_t)((total + 255u) / 256u), count), dim3(256), 0, s, static_cast<const uint8_t *>(raw), raw_stride, nrows, K,
                  static_cast<uint8_t *>(tiled), tiled_stride);
    return hipGetLastError();
}

constexpr uint32_t kIq3SignBytes = 256u * 16u;              // [eight sign bits]: eight fp16 sign masks
constexpr uint32_t kIq3MagBytes = 16u * 512u * 8u;          // [scale nibble][grid entry]: four fp16 magnitudes times 1 + 2 nibble (at most 15 * 31: exact)

__device__ __forceinline__ void build_iq3s_tables(uint8_t *sgn, uint8_t *mag, uint32_t tid, uint32_t nthreads) {
    for (uint32_t e = tid; e < 16u * 512u; e += nthreads) {
        const uint32_t gw = redhip_iq3s_grid[e & 511u];
        const float f = (float)(1u + 2u * (e >> 9));
        uint32_t w2[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const _Float16 lo = (_Float16)(f * (float)((gw >> (16 * i)) & 255u)), hi = (_Float16)(f * (float)((gw >> (16 * i + 8)) & 255u));
            w2[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint2 *>(mag + (size_t)e * 8u) = make_uint2(w2[0], w2[1]);
    }
    for (uint32_t s8 = tid; s8 < 256u; s8 += nthreads) {
        uint32_t w4[4];
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) w4[i] = (((s8 >> (2u * i)) & 1u) << 15) | (((s8 >> (2u * i + 1u)) & 1u) << 31);
        *reinterpret_cast<uint4 *>(sgn + (size_t)s8 * 16u) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
    }
}

// the eight signed, scaled fp16 weights of one word of the tile-major layout
__device__ __forceinline__ half8_t decode_iq3s(uint32_t w, const uint8_t *sgn, const uint8_t *mag) {
    const uint32_t t = (w >> 14) & 0xf000u;                   // scale nibble * 512 entries * 8 bytes
    const uint2 ma = *reinterpret_cast<const uint2 *>(mag + (((w << 3) & 0xff8u) | t));
    const uint2 mb = *reinterpret_cast<const uint2 *>(mag + (((w >> 6) & 0xff8u) | t));
    const uint4 g = *reinterpret_cast<const uint4 *>(sgn + ((w >> 14) & 0xff0u));
    Half8 r;
    r.u = make_uint4(ma.x ^ g.x, ma.y ^ g.y, mb.x ^ g.z, mb.y ^ g.w);
    return r.v;
}

struct Iq3DownArgs {
    PrefillArgs p;                 // act_h / act_l / act_exp (kExpPerPair exponents per pair) from the gate/up kernel, tmp out; routed tiles only
    const uint8_t *experts;        // tile-major IQ3_S down matrices
    uint64_t stride;
};

// Same structure as prefill_down_reg_kernel: wave w computes rows 128 b + 16 w + r of the pass, a tile's activations stay in registers.
template <int NFG>          // ffn = 32 * NFG, NFG <= 16
__global__ __launch_bounds__(kRegWaves * 64) void prefill_down_iq3s_kernel(Iq3DownArgs da) {
    const PrefillArgs &a = da.p;
    constexpr uint32_t F = 32u * NFG, FB = F / 256u, NCK = NFG / 4u;
    __shared__ __attribute__((aligned(16))) uint8_t tables[kIq3SignBytes + kIq3MagBytes];      // static: table reads take immediate offsets
    __shared__ __attribute__((aligned(16))) float pair_scale[kExpPerPair][kTile];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t H = a.hidden;
    const uint8_t *sgn = tables, *mag = tables + kIq3SignBytes;
    build_iq3s_tables(tables, tables + kIq3SignBytes, tid, kRegWaves * 64u);
    const uint32_t T = a.n_tiles[0];
    const uint64_t qs_bytes = (uint64_t)H * NFG * 16u;
    constexpr uint32_t kRowsPerPass = 16u * kRegWaves;
    const uint32_t n_pass_tile = H / kRowsPerPass, parts = n_pass_tile % 4u == 0u ? 4u : n_pass_tile % 2u == 0u ? 2u : 1u, n_pass = n_pass_tile / parts;
    const uint32_t items = T * parts;
    const uint32_t item_begin = (uint32_t)(((uint64_t)blockIdx.x * items) / gridDim.x), item_end = (uint32_t)(((uint64_t)(blockIdx.x + 1u) * items) / gridDim.x);
    Half8 xa[NFG], xb[NFG];
    uint32_t have_tile = 0xffffffffu;
    for (uint32_t item = item_begin; item < item_end; ++item) {
        const uint32_t tile = item / parts, pass0 = (item % parts) * n_pass;
        const uint32_t u = a.tile_group[tile], p0 = a.tile_pair0[tile], n = a.tile_n[tile];
        const uint8_t *dn = da.experts + (uint64_t)a.uid[u] * da.stride;
        if (tile != have_tile) {
            have_tile = tile;
            __syncthreads();
            if (tid < kExpPerPair * kTile && (tid & 3u) < NCK) pair_scale[tid & 3u][tid >> 2] = (tid >> 2) < n ? exp2i(a.act_exp[kExpPerPair * p0 + tid]) : 0.0f;      // IQ3_S: weight = d (1 + 2 nibble) grid, no 1/8
            __syncthreads();
            const uint64_t base = (uint64_t)(p0 + r) * F + 8u * q;
            const bool live = r < n;
#pragma unroll
            for (uint32_t g = 0; g < (uint32_t)NFG; ++g) {
                xa[g].u = make_uint4(0u, 0u, 0u, 0u);
                xb[g].u = xa[g].u;
                if (live) {
                    xa[g].u = *reinterpret_cast<const uint4 *>(a.act_h + base + 32u * g);
                    xb[g].u = *reinterpret_cast<const uint4 *>(a.act_l + base + 32u * g);
                }
            }
        }
        struct Chunk { uint4 w; uint32_t d; };
        auto load_chunk = [&](uint32_t b, uint32_t c) {
            const uint32_t rtile = kRegWaves * (pass0 + b) + wave;
            const uint4 *qp = reinterpret_cast<const uint4 *>(dn + (((uint64_t)rtile * NCK + c) * 16u + r) * 64u + 16u * q);
            const uint16_t *dp = reinterpret_cast<const uint16_t *>(dn + qs_bytes) + ((uint64_t)rtile * FB + c / 2u) * 16u + r;
            return Chunk{qp[0], *dp};
        };
        Chunk cw[NCK];
#pragma unroll
        for (uint32_t c = 0; c < NCK; ++c) cw[c] = load_chunk(0u, c);
#pragma unroll 1
        for (uint32_t b = 0; b < n_pass; ++b) {
            float4_t tot = {0.0f, 0.0f, 0.0f, 0.0f};
            const uint32_t nb = b + 1u < n_pass ? b + 1u : b;          // the last pass reloads itself: no branch around the loads
#pragma unroll
            for (uint32_t c = 0; c < NCK; ++c) {
                const uint32_t w4[4] = {cw[c].w.x, cw[c].w.y, cw[c].w.z, cw[c].w.w};
                const float d = scale_to_f32(cw[c].d);
                cw[c] = load_chunk(nb, c);
                __builtin_amdgcn_sched_barrier(0);         // keeps the loads here: the scheduler otherwise sinks them to the end of the pass
                float4_t hi = {0.0f, 0.0f, 0.0f, 0.0f}, lo = hi;
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) {
                    const uint32_t g = 4u * c + k;
                    const half8_t bw = decode_iq3s(w4[k], sgn, mag);
                    hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[g].v, bw, hi, 0, 0, 0);
                    lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(xb[g].v, bw, lo, 0, 0, 0);
                }
                const float4_t ps = *reinterpret_cast<const float4_t *>(&pair_scale[c][4u * q]);
#pragma unroll
                for (int t = 0; t < 4; ++t) tot[t] = fmaf(fmaf(lo[t], 4.8828125e-4f, hi[t]) * d, ps[t], tot[t]);
            }
            const uint32_t row = kRowsPerPass * (pass0 + b) + 16u * wave + r;
#pragma unroll
            for (uint32_t t = 0; t < 4u; ++t) {
                const uint32_t i = 4u * q + t;
                if (i < n) a.tmp[(uint64_t)(p0 + i) * H + row] = tot[t];
            }
        }
    }
}

// ---------------------------------------------------------------- router logits of a token chunk

// logits[tok][e] = W[e] . x[tok] for an f32 router as a tiled product on v_mfma_f32_16x16x4_f32 (full fp32 multiply-add): a workgroup
// owns 32 rows x 32 tokens, wave (wr, wt) the 16 x 16 block of rows 16 wr .. and tokens 16 wt .. over the whole hidden dimension. Both
// operands pass through LDS in slices of 64 k (double-buffered, one barrier per slice: the next two slices are in registers while this one
// is multiplied), so a row or an activation vector is read from L2 once per workgroup instead of once per 16 x 16 block. Lane
// (r = l % 16, q = l / 16) reads four consecutive k of row r and of token r per 16 k and feeds them to four MFMAs (A[i = r][k = q],
// B[k = q][j = r], D[i = 4q .. 4q + 3][j = r]; the order of k inside a slice does not matter as long as both operands agree). With
// `gate_inp` set, row E is that vector (the shared expert's gate). A second kind of workgroup (blockIdx.x beyond the row tiles,
// launched when xh is set) does the fp16 split of its tokens' activations; it then also multiplies them with the gate vector, so the
// row tiles cover the E matrix rows only (512 experts x 512 tokens: 16 x 16 tiles, one per compute unit, instead of a seventeenth row of
// tiles for the one vector). The same kernel multiplies any f32 matrix [E][H] with a chunk of activations (dense shared expert).
constexpr uint32_t kGemmTile = 32u, kGemmK = 64u, kGemmRow = kGemmK + 4u;      // LDS row of 68 floats: the eight lanes of a 16-byte read pass hit different banks

// Eight waves: waves 0..3 take the even slices of 64 k, waves 4..7 the odd ones (each set one 16 x 16 block per wave, as described above);
// the two partial blocks meet in LDS at the end. Two waves per SIMD, so one's MFMAs run while the other waits at the barrier or for LDS,
// and half as many barriers as slices.
__global__ __launch_bounds__(512) void router_f32_tile_kernel(const float *w, const float *gate_inp, const float *x, float *logits, uint32_t out_stride,
                                                              _Float16 *xh, _Float16 *xl, int *xexp, uint32_t H, uint32_t E, uint32_t ntok) {
    __shared__ __attribute__((aligned(16))) float ws[2][2][kGemmTile][kGemmRow], xs[2][2][kGemmTile][kGemmRow];      // [buffer][k half]
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t n_rows = E + (gate_inp && !xh ? 1u : 0u), row_tiles = (n_rows + kGemmTile - 1u) / kGemmTile, tok_tiles = (ntok + kGemmTile - 1u) / kGemmTile;
    const uint32_t n_tile = row_tiles * tok_tiles;
    if (blockIdx.x >= n_tile) {                            // split job: one wave per token, 8 tokens per workgroup
        const uint32_t tok = 8u * (blockIdx.x - n_tile) + wave;
        if (tok >= ntok) return;
        // the vector as float4 per lane, eight requested at a time (2048 elements per pass: one round trip for the usual widths)
        const float4 *xt = reinterpret_cast<const float4 *>(x + (uint64_t)tok * H), *gv = reinterpret_cast<const float4 *>(gate_inp);
        const uint32_t H4 = H / 4u;
        float amax = 0.0f, gate = 0.0f;
        for (uint32_t base = 0; base < H4; base += 512u) {
            float4 v[8], g[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t i = base + 64u * k + lane;
                v[k] = i < H4 ? xt[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                g[k] = gate_inp && i < H4 ? gv[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                amax = fmaxf(fmaxf(amax, fmaxf(fabsf(v[k].x), fabsf(v[k].y))), fmaxf(fabsf(v[k].z), fabsf(v[k].w)));
                gate = fmaf(g[k].w, v[k].w, fmaf(g[k].z, v[k].z, fmaf(g[k].y, v[k].y, fmaf(g[k].x, v[k].x, gate))));
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { amax = fmaxf(amax, __shfl_xor(amax, o, 64)); gate += __shfl_xor(gate, o, 64); }
        const int e = prescale_exp(amax);
        const float inv = exp2i(-e);
        for (uint32_t base = 0; base < H4; base += 512u) {
            float4 v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) { const uint32_t i = base + 64u * k + lane; v[k] = xt[i < H4 ? i : 0u]; }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t i = base + 64u * k + lane;
                if (i >= H4) continue;
                const float f[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
                half4_t h4, l4;
#pragma unroll
                for (int c = 0; c < 4; ++c) { _Float16 hh, ll; split_hi_lo(f[c], inv, &hh, &ll); h4[c] = hh; l4[c] = ll; }
                *reinterpret_cast<half4_t *>(xh + (uint64_t)tok * H + 4u * i) = h4;
                *reinterpret_cast<half4_t *>(xl + (uint64_t)tok * H + 4u * i) = l4;
            }
        }
        if (lane == 0u) {
            xexp[tok] = e;
            if (gate_inp) logits[(uint64_t)tok * out_stride + E] = gate;
        }
        return;
    }
    // staging: thread t of k half h = t / 256 moves rows (t % 256) / 16 and + 16 of both operands, 16 bytes at column 4 (t % 16) of its half's
    // slice; rows beyond the last one repeat another and are not stored
    // Workgroups are dealt to the eight XCDs in turn, each with its own L2: workgroup i lands on XCD i % 8. The tiles of one XCD form a
    // compact block of the tile grid (a quarter of the row tiles x half of the token tiles), so that an XCD fetches a quarter of the
    // matrix and half of the activations instead of all of both. (A different dealing order would only cost this locality.)
    uint32_t tile_r = blockIdx.x % row_tiles, tile_t = blockIdx.x / row_tiles;
    if (row_tiles % 4u == 0u && tok_tiles % 2u == 0u) {
        const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, br = row_tiles / 4u, bt = tok_tiles / 2u;
        tile_r = (xcd & 3u) * br + slot % br;
        tile_t = (xcd >> 2) * bt + slot / br;
    }
    const uint32_t kh = tid >> 8, srow = (tid & 255u) >> 4, scol = 4u * (tid & 15u);
    const uint32_t row_a = kGemmTile * tile_r + srow, row_b = row_a + 16u, tok_a = kGemmTile * tile_t + srow, tok_b = tok_a + 16u;
    const float *wsrc_a = (row_a < E ? w + (uint64_t)row_a * H : gate_inp ? gate_inp : w) + scol + kh * kGemmK;
    const float *wsrc_b = (row_b < E ? w + (uint64_t)row_b * H : gate_inp ? gate_inp : w) + scol + kh * kGemmK;
    const float *xsrc_a = x + (uint64_t)(tok_a < ntok ? tok_a : ntok - 1u) * H + scol + kh * kGemmK;
    const float *xsrc_b = x + (uint64_t)(tok_b < ntok ? tok_b : ntok - 1u) * H + scol + kh * kGemmK;
    const uint32_t wr = wave & 1u, wt = (wave >> 1) & 1u, n_round = H / (2u * kGemmK);      // hidden is a multiple of 256: an even number of rounds
    constexpr uint32_t kStep = 2u * kGemmK;                // k per round
    // two register sets, one per LDS buffer: the loads of round rd + 2 are issued while round rd is multiplied, so a round trip has two
    // rounds of arithmetic to hide behind (plain variables: arrays of them end up in scratch memory)
    float4 w0a = *reinterpret_cast<const float4 *>(wsrc_a), w0b = *reinterpret_cast<const float4 *>(wsrc_b);
    float4 x0a = *reinterpret_cast<const float4 *>(xsrc_a), x0b = *reinterpret_cast<const float4 *>(xsrc_b);
    float4 w1a = *reinterpret_cast<const float4 *>(wsrc_a + kStep), w1b = *reinterpret_cast<const float4 *>(wsrc_b + kStep);
    float4 x1a = *reinterpret_cast<const float4 *>(xsrc_a + kStep), x1b = *reinterpret_cast<const float4 *>(xsrc_b + kStep);
    float4_t acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = acc0;
    const uint32_t mh = wave >> 2;                         // the k half this wave multiplies
    auto multiply = [&](uint32_t buf) {
#pragma unroll
        for (uint32_t u = 0; u < kGemmK / 16u; ++u) {
            const float4 av = *reinterpret_cast<const float4 *>(&ws[buf][mh][16u * wr + r][16u * u + 4u * q]);
            const float4 bv = *reinterpret_cast<const float4 *>(&xs[buf][mh][16u * wt + r][16u * u + 4u * q]);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, bv.x, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, bv.y, acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, bv.z, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, bv.w, acc1, 0, 0, 0);
        }
    };
    for (uint32_t rd = 0; rd < n_round; rd += 2u) {
        *reinterpret_cast<float4 *>(&ws[0][kh][srow][scol]) = w0a;
        *reinterpret_cast<float4 *>(&ws[0][kh][srow + 16u][scol]) = w0b;
        *reinterpret_cast<float4 *>(&xs[0][kh][srow][scol]) = x0a;
        *reinterpret_cast<float4 *>(&xs[0][kh][srow + 16u][scol]) = x0b;
        __syncthreads();                                   // round rd is in place; the readers of the other buffer (round rd - 1) are past their barrier
        const uint32_t k2 = (rd + 2u < n_round ? rd + 2u : rd) * kStep;          // the last rounds reload themselves: no branch around the loads
        w0a = *reinterpret_cast<const float4 *>(wsrc_a + k2);
        w0b = *reinterpret_cast<const float4 *>(wsrc_b + k2);
        x0a = *reinterpret_cast<const float4 *>(xsrc_a + k2);
        x0b = *reinterpret_cast<const float4 *>(xsrc_b + k2);
        multiply(0u);
        *reinterpret_cast<float4 *>(&ws[1][kh][srow][scol]) = w1a;
        *reinterpret_cast<float4 *>(&ws[1][kh][srow + 16u][scol]) = w1b;
        *reinterpret_cast<float4 *>(&xs[1][kh][srow][scol]) = x1a;
        *reinterpret_cast<float4 *>(&xs[1][kh][srow + 16u][scol]) = x1b;
        __syncthreads();
        const uint32_t k3 = (rd + 3u < n_round ? rd + 3u : rd + 1u) * kStep;
        w1a = *reinterpret_cast<const float4 *>(wsrc_a + k3);
        w1b = *reinterpret_cast<const float4 *>(wsrc_b + k3);
        x1a = *reinterpret_cast<const float4 *>(xsrc_a + k3);
        x1b = *reinterpret_cast<const float4 *>(xsrc_b + k3);
        multiply(1u);
    }
    // the odd slices' blocks go through LDS (buffer 0 was last read two barriers ago) to the waves that hold the even ones
    float *meet = &ws[0][0][0][0];                         // [4 blocks][64 lanes] float4
    __syncthreads();
    if (mh == 1u) *reinterpret_cast<float4 *>(meet + ((wave & 3u) * 64u + lane) * 4u) = make_float4(acc0[0] + acc1[0], acc0[1] + acc1[1], acc0[2] + acc1[2], acc0[3] + acc1[3]);
    __syncthreads();
    if (mh == 1u) return;
    const float4 other = *reinterpret_cast<const float4 *>(meet + (wave * 64u + lane) * 4u);
    const float oth[4] = {other.x, other.y, other.z, other.w};
    const uint32_t out_tok = kGemmTile * tile_t + 16u * wt + r;
#pragma unroll
    for (uint32_t t = 0; t < 4u; ++t) {
        const uint32_t out_row = kGemmTile * tile_r + 16u * wr + 4u * q + t;
        if (out_tok < ntok && out_row < n_rows) logits[(uint64_t)out_tok * out_stride + out_row] = (acc0[t] + acc1[t]) + oth[t];
    }
}

// out[tok][row] = W[row] . x[tok] for an f32 matrix W [n_rows][K] and a chunk of activations x [ntok][K]; extra_row (optional) is one more
// row behind the matrix; xh / xl / xexp (optional): also write the fp16 halves of x
hipError_t launch_f32_tiles(const float *w, const float *extra_row, const float *x, uint32_t ntok, uint32_t K, uint32_t n_rows, float *out,
                            uint32_t out_stride, void *xh, void *xl, int *xexp, hipStream_t s) {
    if (!ntok || !K || K % 256u || !n_rows || !w || !x || !out) return hipErrorInvalidValue;
    const uint32_t row_tiles = (n_rows + (extra_row && !xh ? 1u : 0u) + kGemmTile - 1u) / kGemmTile, tok_tiles = (ntok + kGemmTile - 1u) / kGemmTile;      // (as in the kernel)
    if ((uint64_t)row_tiles * tok_tiles + ntok > 0x7fffffffull) return hipErrorInvalidValue;
    const uint32_t split_wgs = xh ? (ntok + 7u) / 8u : 0u;            // behind the tiles
    REDHIP_LAUNCH(router_f32_tile_kernel, dim3(row_tiles * tok_tiles + split_wgs), dim3(512), 0, s, w, extra_row, x, out, out_stride,
                  static_cast<_Float16 *>(xh), static_cast<_Float16 *>(xl), xexp, K, n_rows, ntok);
    return hipGetLastError();
}

hipError_t launch_router_f32_tiles(const float *w, const float *gate_inp, const float *x, uint32_t ntok, uint32_t hidden, uint32_t n_expert,
                                   float *logits, void *xh, void *xl, int *xexp, hipStream_t s) {
    return launch_f32_tiles(w, gate_inp, x, ntok, hidden, n_expert, logits, n_expert + 1u, xh, xl, xexp, s);
}

// act[tok][c] = silu(gu[tok][c]) * gu[tok][ffn + c]
__global__ void swiglu_rows_kernel(const float *gu, uint32_t gu_stride, uint32_t ffn, float *act) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x, tok = blockIdx.y;
    if (c >= ffn) return;
    const float g = gu[(uint64_t)tok * gu_stride + c], u = gu[(uint64_t)tok * gu_stride + ffn + c];
    act[(uint64_t)tok * ffn + c] = (g / (1.0f + expf(-g))) * u;
}

hipError_t launch_swiglu_rows(const float *gu, uint32_t gu_stride, uint32_t ntok, uint32_t ffn, float *act, hipStream_t s) {
    REDHIP_LAUNCH(swiglu_rows_kernel, dim3((ffn + 255u) / 256u, ntok), dim3(256), 0, s, gu, gu_stride, ffn, act);
    return hipGetLastError();
}

// list_stride: distance of the tile lists in the tile arrays (build_tiles_kernel). hidden >= 1024: wide and narrow tiles in one launch;
// hidden 512: list 0 on the kernel for 16 pairs.
static hipError_t launch_gateup_reg(const TiledArgs &ta, dim3 grid, hipStream_t s, uint32_t list_stride, uint32_t fmt = 0u) {
    const uint32_t hidden = ta.p.hidden;
    hipError_t e = hipSuccess;
    prof_set_stage(ST_PREFILL_GATEUP);
    if (hidden / 512u == 2u || hidden / 512u == 4u) {
#define REDHIP_PGW_ONE(NKC, FMT)                                                                                                          \
    do {                                                                                                                                  \
        static bool attr = false;                                                                                                          \
        if (!attr) {                                                                                                                       \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(prefill_gateup_mixed_kernel<NKC, FMT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideLds); \
            if (e != hipSuccess) return e;                                                                                                 \
            attr = true;                                                                                                                   \
        }                                                                                                                                  \
        REDHIP_LAUNCH((prefill_gateup_mixed_kernel<NKC, FMT>), grid, dim3(kRegWaves * 64), kWideLds, s, ta, list_stride);                  \
    } while (0)
#define REDHIP_PGW(NKC)                                                                                                                   \
    do {                                                                                                                                  \
        if (fmt == 1u) REDHIP_PGW_ONE(NKC, 1);                                                                                             \
        else if (fmt == 2u) REDHIP_PGW_ONE(NKC, 2);                                                                                        \
        else REDHIP_PGW_ONE(NKC, 0);                                                                                                       \
    } while (0)
        if (hidden / 512u == 2u) REDHIP_PGW(2); else REDHIP_PGW(4);
#undef REDHIP_PGW
#undef REDHIP_PGW_ONE
        return hipGetLastError();
    }
    const size_t acts_lds = kNarrowLds;
#define REDHIP_PGR_ONE(NKC, FMT)                                                                                                          \
    do {                                                                                                                                  \
        static bool attr = false;                                                                                                          \
        if (!attr) {                                                                                                                       \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(prefill_gateup_reg_kernel<NKC, FMT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kNarrowLds); \
            if (e != hipSuccess) return e;                                                                                                 \
            attr = true;                                                                                                                   \
        }                                                                                                                                  \
        REDHIP_LAUNCH((prefill_gateup_reg_kernel<NKC, FMT>), grid, dim3(kRegWaves * 64), acts_lds, s, ta);                                 \
    } while (0)
#define REDHIP_PGR(NKC)                                                                                                                   \
    do {                                                                                                                                  \
        if (fmt == 1u) REDHIP_PGR_ONE(NKC, 1);                                                                                             \
        else if (fmt == 2u) REDHIP_PGR_ONE(NKC, 2);                                                                                        \
        else REDHIP_PGR_ONE(NKC, 0);                                                                                                       \
    } while (0)
    switch (hidden / 512u) {
        case 1: REDHIP_PGR(1); break;
        case 2: REDHIP_PGR(2); break;
        case 4: REDHIP_PGR(4); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_PGR
#undef REDHIP_PGR_ONE
    return hipGetLastError();
}

// routed gate/up + SwiGLU of a chunk on the tile-major copy of packed IQ2_XXS gate/up matrices: the front half of a layer whose other
// matrices are of other types. Activations out as f32 [pairs][ffn] (`act`, for kernels on raw rows) or, with act == nullptr, as fp16 halves
// with two exponents per pair (for launch_prefill_down_iq3s). Needs the pair grouping; builds the tile list; the shared expert is not touched.
// Persistent workgroups of the tile kernels: a tile is cut into up to four work items, so small chunks fill more workgroups than they
// have tiles (17 tokens: 152 tiles, 608 items - three rounds on 256 workgroups instead of four on 183)
static inline uint32_t tile_grid(uint32_t tile_bound) { return 4u * tile_bound < 256u ? 4u * tile_bound : 256u; }

hipError_t launch_prefill_gateup_tiled(const void *tiled_experts, uint64_t stride, const uint32_t *uid, const uint32_t *expert_start,
                                       const uint32_t *pair_token, const uint32_t *n_unique, uint32_t *tile_group, uint32_t *tile_pair0, uint32_t *tile_n,
                                       uint32_t *n_tiles, const void *xh, const void *xl, const int *xexp, float *act, void *act_h, void *act_l,
                                       int *act_exp, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert, hipStream_t s, bool tiles_built) {
    if (!fused_iq2_supported(hidden, ffn) || hidden / 512u > 4u || ffn > 512u || !ntok || !tiled_experts || (!act && (!act_h || !act_l || !act_exp)))
        return hipErrorInvalidValue;
    const uint32_t P = ntok * top_k;
    hipError_t e = hipSuccess;
    if (!tiles_built) {
        prof_set_stage(ST_GROUP);
        const TileLists tl{tile_group, tile_pair0, tile_n, n_tiles, prefill_tile_bound(ntok, top_k, n_expert), 0u};      // no shared tiles
        REDHIP_LAUNCH(build_tiles_kernel, dim3(1), dim3(1024), 0, s, expert_start, n_unique, P, tl);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    PrefillArgs a{nullptr, stride, nullptr, uid, pair_token, n_unique, tile_group, tile_pair0, tile_n, n_tiles, static_cast<const _Float16 *>(xh),
                  static_cast<const _Float16 *>(xl), xexp, static_cast<_Float16 *>(act_h), static_cast<_Float16 *>(act_l), act_exp, nullptr, nullptr, hidden,
                  ffn, top_k, ntok};
    const TiledArgs ta{a, static_cast<const uint8_t *>(tiled_experts), nullptr, act, nullptr, 0u};
    const uint32_t tile_bound = prefill_tile_bound(ntok, top_k, n_expert);
    return launch_gateup_reg(ta, dim3(tile_grid(tile_bound)), s, tile_bound);
}

// The routed gate/up and down matrices of a chunk on a layout whose experts are IQ2_XS / IQ1_M: the same tile kernels on the row-major
// streams of the format (gate | up per expert at `packed`, the down matrix at `down`), decoded through the caller's codebooks. The
// tile list is built here (no shared tiles); outputs as the IQ2_XXS tile kernels: fp16 activations per pair, then tmp [pairs][hidden].
hipError_t launch_prefill_streams(uint32_t gate_up_type, const int8_t *gate_up_grid, const void *packed, uint64_t packed_stride, uint32_t down_type,
                                  const int8_t *down_grid, const void *down, uint64_t down_stride, const uint32_t *uid, const uint32_t *expert_start,
                                  const uint32_t *pair_token, const uint32_t *n_unique, uint32_t *tile_group, uint32_t *tile_pair0, uint32_t *tile_n,
                                  uint32_t *n_tiles, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l, int *act_exp, float *tmp,
                                  uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert, hipStream_t s, bool tiles_built) {
    const auto fmt_of = [](uint32_t t) { return t == T_IQ2_XS ? 1u : t == T_IQ1_M ? 2u : 0u; };
    const uint32_t fg = fmt_of(gate_up_type), fd = fmt_of(down_type);
    if (!fg || !fd || !gate_up_grid || !down_grid || !packed || !down || !fused_iq2_supported(hidden, ffn) || hidden / 512u > 4u || (ffn != 256u && ffn != 512u) || !ntok)
        return hipErrorInvalidValue;
    const uint32_t P = ntok * top_k;
    hipError_t e = hipSuccess;
    if (!tiles_built) {
        prof_set_stage(ST_GROUP);
        const TileLists tl{tile_group, tile_pair0, tile_n, n_tiles, prefill_tile_bound(ntok, top_k, n_expert), 0u};      // no shared tiles
        REDHIP_LAUNCH(build_tiles_kernel, dim3(1), dim3(1024), 0, s, expert_start, n_unique, P, tl);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    PrefillArgs a{nullptr, packed_stride, nullptr, uid, pair_token, n_unique, tile_group, tile_pair0, tile_n, n_tiles, static_cast<const _Float16 *>(xh),
                  static_cast<const _Float16 *>(xl), xexp, static_cast<_Float16 *>(act_h), static_cast<_Float16 *>(act_l), act_exp, tmp, nullptr, hidden,
                  ffn, top_k, ntok};
    const uint32_t tile_bound = prefill_tile_bound(ntok, top_k, n_expert);
    const dim3 grid(tile_grid(tile_bound)), rblock(kRegWaves * 64);
    const TiledArgs tg{a, static_cast<const uint8_t *>(packed), nullptr, nullptr, gate_up_grid, 0u};
    e = launch_gateup_reg(tg, grid, s, tile_bound, fg);
    if (e != hipSuccess) return e;
    a.stride = down_stride;
    const TiledArgs td{a, static_cast<const uint8_t *>(down), nullptr, nullptr, down_grid, 0u};
    prof_set_stage(ST_PREFILL_DOWN);
    if (ffn == 256u) {
        if (fd == 1u) REDHIP_LAUNCH((prefill_down_reg_kernel<8, 3>), grid, rblock, 0, s, td);      // (IQ2_XS: the scale-folded table, 130 KB of LDS)
        else REDHIP_LAUNCH((prefill_down_reg_kernel<8, 2>), grid, rblock, 0, s, td);
    } else {
        if (fd == 1u) REDHIP_LAUNCH((prefill_down_reg_kernel<16, 3>), grid, rblock, 0, s, td);
        else REDHIP_LAUNCH((prefill_down_reg_kernel<16, 2>), grid, rblock, 0, s, td);
    }
    return hipGetLastError();
}

// routed down projection of a chunk on tile-major IQ3_S matrices, behind launch_prefill_gateup_tiled (its tile list and fp16 activations)
hipError_t launch_prefill_down_iq3s(const void *tiled_down, uint64_t stride, const uint32_t *uid, const uint32_t *n_unique, const uint32_t *tile_group,
                                    const uint32_t *tile_pair0, const uint32_t *tile_n, const uint32_t *n_tiles, const void *act_h, const void *act_l,
                                    const int *act_exp, float *tmp, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok, uint32_t n_expert,
                                    hipStream_t s) {
    if (!tiled_down || !hidden || hidden % 128u || (ffn != 256u && ffn != 512u) || !ntok) return hipErrorInvalidValue;
    PrefillArgs a{nullptr, stride, nullptr, uid, nullptr, n_unique, tile_group, tile_pair0, tile_n, n_tiles, nullptr, nullptr, nullptr,
                  static_cast<_Float16 *>(const_cast<void *>(act_h)), static_cast<_Float16 *>(const_cast<void *>(act_l)), const_cast<int *>(act_exp), tmp,
                  nullptr, hidden, ffn, top_k, ntok};
    const Iq3DownArgs da{a, static_cast<const uint8_t *>(tiled_down), stride};
    const uint32_t tile_bound = prefill_tile_bound(ntok, top_k, n_expert);
    const dim3 grid(tile_grid(tile_bound));
    prof_set_stage(ST_PREFILL_DOWN);
    if (ffn == 256u) REDHIP_LAUNCH(prefill_down_iq3s_kernel<8>, grid, dim3(kRegWaves * 64), 0, s, da);
    else REDHIP_LAUNCH(prefill_down_iq3s_kernel<16>, grid, dim3(kRegWaves * 64), 0, s, da);
    return hipGetLastError();
}

hipError_t launch_prefill_packed(const void *experts, uint64_t stride, const void *shared, const void *tiled_experts, const void *tiled_shared,
                                 const uint32_t *uid, const uint32_t *expert_start,
                                 const uint32_t *pair_token, const uint32_t *n_unique, uint32_t *tile_group, uint32_t *tile_pair0,
                                 uint32_t *tile_n, uint32_t *n_tiles, const void *xh, const void *xl, const int *xexp, void *act_h, void *act_l,
                                 int *act_exp, float *tmp, float *sh_tmp, uint32_t hidden, uint32_t ffn, uint32_t top_k, uint32_t ntok,
                                 uint32_t n_expert, hipStream_t s, bool tiles_built, bool with_shared) {
    if (!fused_iq2_supported(hidden, ffn) || hidden / 512u > 4u || !ntok) return hipErrorInvalidValue;
    const uint32_t P = ntok * top_k;
    hipError_t e = hipSuccess;
    if (!tiles_built) {
        prof_set_stage(ST_GROUP);
        const TileLists tl{tile_group, tile_pair0, tile_n, n_tiles, prefill_tile_bound(ntok, top_k, n_expert), with_shared ? ntok : 0u};
        REDHIP_LAUNCH(build_tiles_kernel, dim3(1), dim3(1024), 0, s, expert_start, n_unique, P, tl);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    PrefillArgs a{static_cast<const uint8_t *>(experts), stride, static_cast<const uint8_t *>(shared), uid, pair_token, n_unique,
                  tile_group, tile_pair0, tile_n, n_tiles, static_cast<const _Float16 *>(xh), static_cast<const _Float16 *>(xl), xexp,
                  static_cast<_Float16 *>(act_h), static_cast<_Float16 *>(act_l), act_exp, tmp, sh_tmp, hidden, ffn, top_k, ntok};
    const uint32_t tile_bound = prefill_tile_bound(ntok, top_k, n_expert);
    const dim3 grid(tile_bound < 256u ? tile_bound : 256u), block(kWaves * 64);
    if (tiled_experts && (tiled_shared || !with_shared) && ffn <= 512u) {          // tile-major copy present: activations of a tile in registers
        const TiledArgs ta{a, static_cast<const uint8_t *>(tiled_experts), static_cast<const uint8_t *>(tiled_shared), nullptr, nullptr, 0u};
        const dim3 rblock(kRegWaves * 64), rgrid(tile_grid(tile_bound));
        e = launch_gateup_reg(ta, rgrid, s, tile_bound);
        if (e != hipSuccess) return e;
        prof_set_stage(ST_PREFILL_DOWN);
        if (ffn == 256u) REDHIP_LAUNCH((prefill_down_reg_kernel<8, 0>), rgrid, rblock, 0, s, ta);
        else REDHIP_LAUNCH((prefill_down_reg_kernel<16, 0>), rgrid, rblock, 0, s, ta);
        return hipGetLastError();
    }
    const size_t dyn_lds = (size_t)2u * kTile * (hidden + kRowPad) * 2u;
    prof_set_stage(ST_PREFILL_GATEUP);
#define REDHIP_PGU(NKC)                                                                                                                   \
    do {                                                                                                                                  \
        static bool attr = false;                                                                                                          \
        if (!attr) {                                                                                                                       \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(prefill_gateup_kernel<NKC>), hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024); \
            if (e != hipSuccess) return e;                                                                                                 \
            attr = true;                                                                                                                   \
        }                                                                                                                                  \
        REDHIP_LAUNCH(prefill_gateup_kernel<NKC>, grid, block, dyn_lds, s, a);                                                             \
    } while (0)
    switch (hidden / 512u) {
        case 1: REDHIP_PGU(1); break;
        case 2: REDHIP_PGU(2); break;
        case 4: REDHIP_PGU(4); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_PGU
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    prof_set_stage(ST_PREFILL_DOWN);
    const size_t down_lds = (size_t)2u * kTile * (ffn + kRowPad) * 2u;
#define REDHIP_PDN(NFG)                                                                                                                   \
    do {                                                                                                                                  \
        static bool attr = false;                                                                                                          \
        if (!attr) {                                                                                                                       \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(prefill_down_kernel<NFG>), hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024); \
            if (e != hipSuccess) return e;                                                                                                 \
            attr = true;                                                                                                                   \
        }                                                                                                                                  \
        REDHIP_LAUNCH(prefill_down_kernel<NFG>, grid, block, down_lds, s, a);                                                              \
    } while (0)
    switch (ffn / 256u) {
        case 1: REDHIP_PDN(8); break;
        case 2: REDHIP_PDN(16); break;
        case 3: REDHIP_PDN(24); break;
        case 4: REDHIP_PDN(32); break;
        default: return hipErrorInvalidValue;
    }
#undef REDHIP_PDN
    return hipGetLastError();
}

}  // namespace redhip
