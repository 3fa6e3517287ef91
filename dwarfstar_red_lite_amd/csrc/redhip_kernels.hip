// gfx950 kernels over raw GGUF rows: dequantisation, GEMV, router selection, token grouping, and the
// single-token expert FFN (gate/up/SwiGLU, then down fused with the weighted combine and the shared expert).
// Wavefronts are 64 wide; a row is split over LPR lanes (8..64), each lane taking 32-weight chunks, and the
// partial sums meet in a butterfly of cross-lane shuffles.
#include "redhip_decode.h"

#include <string.h>

#include <mutex>
#include <vector>

namespace redhip {

// the codebooks are constant device arrays of this translation unit (redhip_tables.h): nothing to upload
static inline hipError_t ensure_tables() { return hipSuccess; }

static inline uint32_t lanes_per_row(uint32_t ncols) {
    const uint32_t chunks = ncols / 32u;
    return chunks >= 64u ? 64u : chunks >= 32u ? 32u : chunks >= 16u ? 16u : 8u;
}
// x staged in LDS with one pad word per 32 floats, so lanes that walk different chunks hit different banks
__device__ __forceinline__ uint32_t pad32(uint32_t i) { return i + (i >> 5); }
static inline uint32_t padded_floats(uint32_t n) { return n + (n >> 5); }

// ---------------------------------------------------------------- IQ2_XS / IQ1_M (caller-supplied codebooks)

// The reference hands these codebooks to its kernels as arguments (native/redmetal_ffn.m:223-227); here they live in
// device memory of this translation unit, uploaded by the pool / one-shot / resident-layer surfaces.
__device__ __attribute__((aligned(16))) int8_t g_iq2xs_grid[512 * 8];
__device__ __attribute__((aligned(16))) int8_t g_iq1m_grid[2048 * 8];

// One pair of tables per process. Pools and resident layers that decode through them bind to their content; while any is bound,
// an upload of different content is refused (the bound users would silently decode through the wrong tables), an upload of the same
// content is free. With nobody bound an upload replaces the tables.
static std::mutex g_grid_mu;
static std::vector<int8_t> g_grid_host[2];      // what the device holds: IQ2_XS, IQ1_M (empty: never uploaded)
static std::vector<const void *> g_grid_bound;  // the owners bound to that content

std::mutex &caller_grid_mutex() { return g_grid_mu; }

bool caller_grid_present(uint32_t type) {
    std::lock_guard<std::mutex> lk(g_grid_mu);
    return type == T_IQ2_XS ? !g_grid_host[0].empty() : type == T_IQ1_M ? !g_grid_host[1].empty() : true;
}

static bool grid_is_bound(const void *owner) {
    for (const void *o : g_grid_bound) if (o == owner) return true;
    return false;
}

hipError_t set_caller_grids_locked(const int8_t *iq2_xs, const int8_t *iq1_m, const void *bind_owner) {
    if (bind_owner && grid_is_bound(bind_owner)) return hipSuccess;
    const int8_t *src[2] = {iq2_xs, iq1_m};
    const size_t n[2] = {sizeof(g_iq2xs_grid), sizeof(g_iq1m_grid)};
    bool differs[2] = {false, false};
    for (int k = 0; k < 2; ++k)
        differs[k] = src[k] && (g_grid_host[k].size() != n[k] || memcmp(g_grid_host[k].data(), src[k], n[k]) != 0);
    if ((differs[0] || differs[1]) && !g_grid_bound.empty()) return hipErrorContextAlreadyInUse;      // see caller_grid_conflict()
    hipError_t e = hipSuccess;
    if (differs[0]) e = hipMemcpyToSymbol(HIP_SYMBOL(g_iq2xs_grid), iq2_xs, n[0]);
    if (e == hipSuccess && differs[0]) g_grid_host[0].assign(iq2_xs, iq2_xs + n[0]);
    if (e == hipSuccess && differs[1]) e = hipMemcpyToSymbol(HIP_SYMBOL(g_iq1m_grid), iq1_m, n[1]);
    if (e == hipSuccess && differs[1]) g_grid_host[1].assign(iq1_m, iq1_m + n[1]);
    if (e == hipSuccess && bind_owner) g_grid_bound.push_back(bind_owner);
    return e;
}

hipError_t set_caller_grids(const int8_t *iq2_xs, const int8_t *iq1_m, const void *bind_owner) {
    std::lock_guard<std::mutex> lk(g_grid_mu);
    return set_caller_grids_locked(iq2_xs, iq1_m, bind_owner);
}

bool caller_grids_bound(const void *owner) {
    std::lock_guard<std::mutex> lk(g_grid_mu);
    return grid_is_bound(owner);
}

void forget_caller_grids(const void *owner) {
    std::lock_guard<std::mutex> lk(g_grid_mu);
    for (size_t i = 0; i < g_grid_bound.size(); ++i)
        if (g_grid_bound[i] == owner) { g_grid_bound.erase(g_grid_bound.begin() + (long)i); break; }
}

template <> __device__ __forceinline__ void decode32<T_IQ2_XS>(const uint8_t *row, uint32_t chunk, float *w) { decode32_cb<T_IQ2_XS>(row, chunk, w, g_iq2xs_grid); }
template <> __device__ __forceinline__ void decode32<T_IQ1_M>(const uint8_t *row, uint32_t chunk, float *w) { decode32_cb<T_IQ1_M>(row, chunk, w, g_iq1m_grid); }

// device address of the codebook the process holds for `type` (nullptr: the type has none)
const int8_t *caller_grid_device(uint32_t type) {
    void *p = nullptr;
    if (type == T_IQ2_XS) { if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_iq2xs_grid)) != hipSuccess) return nullptr; }
    else if (type == T_IQ1_M) { if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_iq1m_grid)) != hipSuccess) return nullptr; }
    return static_cast<const int8_t *>(p);
}

template <uint32_t T>
__device__ __forceinline__ float chunk_dot(const uint8_t *row, uint32_t chunk, const float *x33) {
    float w[32];
    decode32<T>(row, chunk, w);
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) acc = fmaf(w[j], x33[j], acc);
    return acc;
}

template <int LPR> __device__ __forceinline__ float sub_reduce(float v) {
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// ---------------------------------------------------------------- dequantisation (parity tap)

template <uint32_t T>
__global__ __launch_bounds__(256) void dequant_rows_kernel(const uint8_t *rows, uint64_t rb, uint32_t nrows, uint32_t chunks_per_row, float *out) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (gid >= (uint64_t)nrows * chunks_per_row) return;
    const uint32_t r = (uint32_t)(gid / chunks_per_row), c = (uint32_t)(gid % chunks_per_row);
    float w[32];
    decode32<T>(rows + (uint64_t)r * rb, c, w);
    float4 *o = reinterpret_cast<float4 *>(out + ((uint64_t)r * chunks_per_row + c) * 32u);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = make_float4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
}

hipError_t launch_dequant_rows(uint32_t type, const void *rows, uint32_t nrows, uint32_t ncols, float *out, hipStream_t s) {
    hipError_t e = ensure_tables();
    if (e != hipSuccess) return e;
    const uint64_t rb = pool_row_bytes(type, ncols);
    if (!rb || ncols % 32u || !nrows) return hipErrorInvalidValue;
    const uint32_t cpr = ncols / 32u;
    const uint64_t total = (uint64_t)nrows * cpr;
    const dim3 grid((uint32_t)((total + 255u) / 256u));
    const uint8_t *p = static_cast<const uint8_t *>(rows);
    switch (type) {
        case T_IQ2_XXS: REDHIP_LAUNCH(dequant_rows_kernel<T_IQ2_XXS>, dim3(grid), dim3(256), 0, s, p, rb, nrows, cpr, out); break;
        case T_IQ3_S: REDHIP_LAUNCH(dequant_rows_kernel<T_IQ3_S>, dim3(grid), dim3(256), 0, s, p, rb, nrows, cpr, out); break;
        case T_Q6_K: REDHIP_LAUNCH(dequant_rows_kernel<T_Q6_K>, dim3(grid), dim3(256), 0, s, p, rb, nrows, cpr, out); break;
        case T_F32: REDHIP_LAUNCH(dequant_rows_kernel<T_F32>, dim3(grid), dim3(256), 0, s, p, rb, nrows, cpr, out); break;
        case T_IQ2_XS: REDHIP_LAUNCH(dequant_rows_kernel<T_IQ2_XS>, dim3(grid), dim3(256), 0, s, p, rb, nrows, cpr, out); break;
        case T_IQ1_M: REDHIP_LAUNCH(dequant_rows_kernel<T_IQ1_M>, dim3(grid), dim3(256), 0, s, p, rb, nrows, cpr, out); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------- GEMV over raw rows

// x is read straight from global memory: the lanes of a row take consecutive 128-byte pieces, so a wave's read is one contiguous
// run, it is issued together with the weight loads, and there is no staging barrier in front of the first decode
template <uint32_t T, int LPR>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const uint8_t *w, uint64_t rb, uint32_t ncols, uint32_t row_start,
                                                        uint32_t row_count, const float *x, float *out) {
    const uint32_t sub = threadIdx.x % LPR, r = blockIdx.x * (blockDim.x / LPR) + threadIdx.x / LPR;
    float acc = 0.0f;
    if (r < row_count) {
        const uint8_t *row = w + (uint64_t)(row_start + r) * rb;
        for (uint32_t c = sub; c < ncols / 32u; c += LPR) {
            float xv[32];
            const float4 *xp = reinterpret_cast<const float4 *>(x + 32u * c);
#pragma unroll
            for (int i = 0; i < 8; ++i) { const float4 v = xp[i]; xv[4 * i] = v.x; xv[4 * i + 1] = v.y; xv[4 * i + 2] = v.z; xv[4 * i + 3] = v.w; }
            acc += chunk_dot<T>(row, c, xv);
        }
    }
    acc = sub_reduce<LPR>(acc);
    if (sub == 0u && r < row_count) out[r] = acc;
}

// IQ2_XXS rows of at least 2048 columns: the same sums in the same order with the grid in LDS. The lanes request their grid entries
// together with their weights and activations, so the launch waits for device memory once; decode32 looks the grid up in device
// memory with indices that come from the weights, a second round trip behind the first.
// One wave per row, kGemvLdsWaves rows per workgroup.
constexpr uint32_t kGemvLdsWaves = 2u;      // (512 rows of 2048 columns back to back: 2.84 us per launch; one wave per workgroup 2.85, four 3.08)
__global__ __launch_bounds__(kGemvLdsWaves * 64) void gemv_iq2xxs_lds_kernel(const uint8_t *w, uint64_t rb, uint32_t ncols, uint32_t row_start, uint32_t row_count,
                                                                            const float *x, float *out) {
    __shared__ __attribute__((aligned(16))) uint64_t grid_lds[256];
    const uint32_t tid = threadIdx.x, sub = tid & 63u, r = blockIdx.x * kGemvLdsWaves + (tid >> 6);
    constexpr uint32_t kSeeds = 256u / (kGemvLdsWaves * 64u);      // grid entries per lane
    uint64_t seed[kSeeds];
#pragma unroll
    for (uint32_t i = 0; i < kSeeds; ++i) seed[i] = redhip_iq2xxs_grid[kSeeds * tid + i];
    const uint32_t rr = r < row_count ? r : row_count - 1u;      // (every lane reaches the barrier; a surplus wave repeats the last row and stores nothing)
    const uint8_t *row = w + (uint64_t)(row_start + rr) * rb;
    float acc = 0.0f;
    bool table_ready = false;
    for (uint32_t c = sub; c < ncols / 32u; c += 64u) {
        const uint8_t *bp = row + (size_t)(c >> 3) * 66u;
        const uint32_t g = c & 7u;
        const uint32_t dbits = ld_u16(bp), idx4 = ld_u32_a2(bp + 2u + 8u * g), aux = ld_u32_a2(bp + 6u + 8u * g);
        float xv[32];
        const float4 *xp = reinterpret_cast<const float4 *>(x + 32u * c);
#pragma unroll
        for (int i = 0; i < 8; ++i) { const float4 v = xp[i]; xv[4 * i] = v.x; xv[4 * i + 1] = v.y; xv[4 * i + 2] = v.z; xv[4 * i + 3] = v.w; }
        if (!table_ready) {
#pragma unroll
            for (uint32_t i = 0; i < kSeeds; ++i) grid_lds[kSeeds * tid + i] = seed[i];
            __syncthreads();
            table_ready = true;
        }
        const float db = half_bits_to_f32(dbits) * (0.5f + (float)(aux >> 28)) * 0.25f;
        float part = 0.0f;
#pragma unroll
        for (uint32_t l = 0; l < 4u; ++l) {
            const uint64_t mag = grid_lds[(idx4 >> (8u * l)) & 255u];
            const uint32_t s7 = (aux >> (7u * l)) & 127u;
            const uint32_t s8 = s7 | ((__popc(s7) & 1u) << 7);
#pragma unroll
            for (uint32_t j = 0; j < 8u; ++j)
                part = fmaf(apply_sign(db * (float)((uint32_t)(mag >> (8u * j)) & 255u), (s8 >> j) & 1u), xv[8u * l + j], part);
        }
        acc += part;
    }
    acc = sub_reduce<64>(acc);
    if (sub == 0u && r < row_count) out[r] = acc;
}

template <uint32_t T>
static hipError_t gemv_dispatch(const uint8_t *w, uint32_t ncols, uint32_t row_start, uint32_t row_count, const float *x, float *out, hipStream_t s) {
    const uint64_t rb = pool_row_bytes(T, ncols);
    const uint32_t lpr = lanes_per_row(ncols);
    if constexpr (T == T_IQ2_XXS) {
        if (lpr == 64u) {
            REDHIP_LAUNCH(gemv_iq2xxs_lds_kernel, dim3((row_count + kGemvLdsWaves - 1u) / kGemvLdsWaves), dim3(kGemvLdsWaves * 64u), 0, s, w, rb, ncols, row_start, row_count, x, out);
            return hipGetLastError();
        }
    }
    // one wave per workgroup while that still leaves fewer workgroups than twice the compute units
    const uint32_t nt = (row_count + 256u / lpr - 1u) / (256u / lpr) < 512u ? 64u : 256u;
    const dim3 grid((row_count + nt / lpr - 1u) / (nt / lpr));
    switch (lpr) {
        case 64: REDHIP_LAUNCH((gemv_rows_kernel<T, 64>), dim3(grid), dim3(nt), 0, s, w, rb, ncols, row_start, row_count, x, out); break;
        case 32: REDHIP_LAUNCH((gemv_rows_kernel<T, 32>), dim3(grid), dim3(nt), 0, s, w, rb, ncols, row_start, row_count, x, out); break;
        case 16: REDHIP_LAUNCH((gemv_rows_kernel<T, 16>), dim3(grid), dim3(nt), 0, s, w, rb, ncols, row_start, row_count, x, out); break;
        default: REDHIP_LAUNCH((gemv_rows_kernel<T, 8>), dim3(grid), dim3(nt), 0, s, w, rb, ncols, row_start, row_count, x, out); break;
    }
    return hipGetLastError();
}

hipError_t launch_gemv_rows(uint32_t type, const void *w, uint32_t ncols, uint32_t row_start, uint32_t row_count,
                            const float *x, float *out, hipStream_t s) {
    hipError_t e = ensure_tables();
    if (e != hipSuccess) return e;
    if (!pool_row_bytes(type, ncols) || ncols % 256u || !row_count || (reinterpret_cast<uintptr_t>(x) & 15u)) return hipErrorInvalidValue;      // x is read as float4
    const uint8_t *p = static_cast<const uint8_t *>(w);
    switch (type) {
        case T_IQ2_XXS: return gemv_dispatch<T_IQ2_XXS>(p, ncols, row_start, row_count, x, out, s);
        case T_IQ3_S: return gemv_dispatch<T_IQ3_S>(p, ncols, row_start, row_count, x, out, s);
        case T_Q6_K: return gemv_dispatch<T_Q6_K>(p, ncols, row_start, row_count, x, out, s);
        case T_F32: return gemv_dispatch<T_F32>(p, ncols, row_start, row_count, x, out, s);
        case T_IQ2_XS: return gemv_dispatch<T_IQ2_XS>(p, ncols, row_start, row_count, x, out, s);
        case T_IQ1_M: return gemv_dispatch<T_IQ1_M>(p, ncols, row_start, row_count, x, out, s);
        default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------- SwiGLU

__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.0f + expf(-g))) * u; }

__global__ void silu_mul_kernel(const float *gate, const float *up, float *act, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) act[i] = silu_mul(gate[i], up[i]);
}

hipError_t launch_silu_mul(const float *gate, const float *up, float *act, uint32_t n, hipStream_t s) {
    REDHIP_LAUNCH(silu_mul_kernel, dim3((n + 255u) / 256u), dim3(256), 0, s, gate, up, act, n);
    return hipGetLastError();
}

// ---------------------------------------------------------------- router selection

// One workgroup of 256 lanes per token. Probabilities are formed exactly as the reference does
// (expf(l - max), double sum, one float reciprocal), selection is on the probabilities with ties to the lower
// index, and the k selected weights are renormalised with a double sum taken in selection order.
__global__ __launch_bounds__(256) void route_select_kernel(const float *logits, uint32_t n_expert, uint32_t top_k,
                                                           uint32_t *ids, float *weights, float *probs,
                                                           const float *gate_inp, const float *x, uint32_t hidden, float *scalar) {
    __shared__ float p[1024];
    __shared__ float red_f[4];
    __shared__ double red_d[4];
    __shared__ uint32_t red_i[4];
    __shared__ float sel_p[16];
    __shared__ uint32_t sel_i[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, tok = blockIdx.x;
    const float *l = logits + (uint64_t)tok * n_expert;

    float m = -INFINITY;
    for (uint32_t i = tid; i < n_expert; i += 256u) m = fmaxf(m, l[i]);
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if (lane == 0u) red_f[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red_f[0], red_f[1]), fmaxf(red_f[2], red_f[3]));

    double part = 0.0;
    for (uint32_t i = tid; i < n_expert; i += 256u) {
        const float e = expf(l[i] - m);
        p[i] = e;
        part += (double)e;
    }
    for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
    if (lane == 0u) red_d[wave] = part;
    __syncthreads();
    const double denom = (red_d[0] + red_d[1]) + (red_d[2] + red_d[3]);
    const bool bad = !(denom > 0.0) || isinf(denom) || isnan(denom);
    const float inv = bad ? 0.0f : (float)(1.0 / denom);
    for (uint32_t i = tid; i < n_expert; i += 256u) {
        const float v = p[i] * inv;
        p[i] = v;
        if (probs) probs[(uint64_t)tok * n_expert + i] = v;
    }
    __syncthreads();

    for (uint32_t k = 0; k < top_k; ++k) {
        float bp = -INFINITY;
        uint32_t bi = 0xffffffffu;
        for (uint32_t i = tid; i < n_expert; i += 256u) {
            const float v = p[i];                       // taken entries hold -1
            if (v >= 0.0f && (v > bp || (v == bp && i < bi))) { bp = v; bi = i; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float op = __shfl_xor(bp, o, 64);
            const uint32_t oi = __shfl_xor(bi, o, 64);
            if (oi != 0xffffffffu && (bi == 0xffffffffu || op > bp || (op == bp && oi < bi))) { bp = op; bi = oi; }
        }
        if (lane == 0u) { red_f[wave] = bp; red_i[wave] = bi; }
        __syncthreads();
        if (tid == 0u) {
            float fp = red_f[0];
            uint32_t fi = red_i[0];
            for (int w = 1; w < 4; ++w) {
                const float op = red_f[w];
                const uint32_t oi = red_i[w];
                if (oi != 0xffffffffu && (fi == 0xffffffffu || op > fp || (op == fp && oi < fi))) { fp = op; fi = oi; }
            }
            if (fi == 0xffffffffu) { fi = k; fp = 0.0f; }      // only when every probability is NaN: keep ids in range
            sel_p[k] = fp;
            sel_i[k] = fi;
            p[fi] = -1.0f;
        }
        __syncthreads();
    }
    if (tid == 0u) {
        double sum = 0.0;
        for (uint32_t k = 0; k < top_k; ++k) sum += (double)sel_p[k];
        const bool bad2 = bad || !(sum > 0.0) || isinf(sum) || isnan(sum);
        const float invs = bad2 ? __uint_as_float(0x7fc00000u) : (float)(1.0 / sum);
        for (uint32_t k = 0; k < top_k; ++k) {
            ids[(uint64_t)tok * top_k + k] = sel_i[k];
            weights[(uint64_t)tok * top_k + k] = sel_p[k] * invs;      // NaN weights flag an invalid softmax
        }
    }
    if (scalar) {                                        // shared-expert scalar gate sigmoid(gate_inp . x_t)
        const float *xt = x + (uint64_t)tok * hidden;
        double acc = 0.0;
        for (uint32_t i = tid; i < hidden; i += 256u) acc += (double)gate_inp[i] * (double)xt[i];
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
        __syncthreads();
        if (lane == 0u) red_d[wave] = acc;
        __syncthreads();
        if (tid == 0u) {
            const double z = (red_d[0] + red_d[1]) + (red_d[2] + red_d[3]);
            scalar[tok] = (float)(1.0 / (1.0 + exp(-z)));
        }
    }
}

hipError_t launch_route_select(const float *logits, uint32_t ntok, uint32_t n_expert, uint32_t top_k,
                               uint32_t *ids, float *weights, float *probs,
                               const float *gate_inp, const float *x, uint32_t hidden, float *scalar, hipStream_t s) {
    if (!ntok || !n_expert || n_expert > 1024u || !top_k || top_k > 16u || top_k > n_expert) return hipErrorInvalidValue;
    if (scalar && (!gate_inp || !x)) return hipErrorInvalidValue;
    REDHIP_LAUNCH(route_select_kernel, dim3(ntok), dim3(256), 0, s, logits, n_expert, top_k, ids, weights, probs, gate_inp, x, hidden, scalar);
    return hipGetLastError();
}

// ---------------------------------------------------------------- single-token expert FFN

template <uint32_t T, int LPR>
__global__ __launch_bounds__(256) void moe_gateup_kernel(const uint8_t *base, uint64_t stride, uint64_t gate_bytes,
                                                         const uint32_t *ids, uint32_t hidden, uint32_t ffn,
                                                         const float *x, float *act, uint32_t id_limit, uint32_t *status,
                                                         const uint64_t *table, const float *x1, uint32_t x_split) {
    extern __shared__ float xs[];
    const uint32_t slot = blockIdx.y, e = ids ? guarded_id(ids[slot], id_limit, status) : slot;
    const float *xin = x1 && slot >= x_split ? x1 : x;
    for (uint32_t i = threadIdx.x; i < hidden; i += 256u) xs[pad32(i)] = xin[i];
    __syncthreads();
    const uint8_t *ebase = table ? reinterpret_cast<const uint8_t *>(table[slot]) : base + (uint64_t)e * stride;
    const uint32_t sub = threadIdx.x % LPR, r = blockIdx.x * (256u / LPR) + threadIdx.x / LPR;
    const uint64_t rb = (uint64_t)(hidden / 256u) * Fmt<T>::kBlock;
    float g = 0.0f, u = 0.0f;
    if (r < ffn) {
        const uint8_t *grow = ebase + (uint64_t)r * rb;
        const uint8_t *urow = grow + gate_bytes;
        for (uint32_t c = sub; c < hidden / 32u; c += LPR) {
            g += chunk_dot<T>(grow, c, xs + 33u * c);
            u += chunk_dot<T>(urow, c, xs + 33u * c);
        }
    }
    g = sub_reduce<LPR>(g);
    u = sub_reduce<LPR>(u);
    if (sub == 0u && r < ffn) act[(uint64_t)slot * ffn + r] = silu_mul(g, u);
}

template <uint32_t T>
static hipError_t gateup_dispatch(const ExpertSet &ex, const uint32_t *ids, uint32_t n_slot, uint32_t hidden, uint32_t ffn,
                                  const float *x, float *act, hipStream_t s, const float *x1, uint32_t x_split) {
    const uint32_t lpr = lanes_per_row(hidden);
    const dim3 grid((ffn + 256u / lpr - 1u) / (256u / lpr), n_slot);
    const size_t lds = padded_floats(hidden) * sizeof(float);
    switch (lpr) {
        case 64: REDHIP_LAUNCH((moe_gateup_kernel<T, 64>), dim3(grid), dim3(256), lds, s, ex.base, ex.stride, ex.gate_bytes, ids, hidden, ffn, x, act, route_guard().id_limit, route_guard().status, ex.table, x1, x_split); break;
        case 32: REDHIP_LAUNCH((moe_gateup_kernel<T, 32>), dim3(grid), dim3(256), lds, s, ex.base, ex.stride, ex.gate_bytes, ids, hidden, ffn, x, act, route_guard().id_limit, route_guard().status, ex.table, x1, x_split); break;
        case 16: REDHIP_LAUNCH((moe_gateup_kernel<T, 16>), dim3(grid), dim3(256), lds, s, ex.base, ex.stride, ex.gate_bytes, ids, hidden, ffn, x, act, route_guard().id_limit, route_guard().status, ex.table, x1, x_split); break;
        default: REDHIP_LAUNCH((moe_gateup_kernel<T, 8>), dim3(grid), dim3(256), lds, s, ex.base, ex.stride, ex.gate_bytes, ids, hidden, ffn, x, act, route_guard().id_limit, route_guard().status, ex.table, x1, x_split); break;
    }
    return hipGetLastError();
}

hipError_t launch_moe_gateup(const ExpertSet &ex, const uint32_t *ids, uint32_t n_slot, uint32_t hidden, uint32_t ffn,
                             const float *x, float *act, hipStream_t s, const float *x1, uint32_t x_split) {
    hipError_t e = ensure_tables();
    if (e != hipSuccess) return e;
    if (!n_slot || hidden % 256u || ffn % 256u || (size_t)padded_floats(hidden) * 4u > 64u * 1024u) return hipErrorInvalidValue;
    switch (ex.gate_up_type) {
        case T_IQ2_XXS: return gateup_dispatch<T_IQ2_XXS>(ex, ids, n_slot, hidden, ffn, x, act, s, x1, x_split);
        case T_IQ3_S: return gateup_dispatch<T_IQ3_S>(ex, ids, n_slot, hidden, ffn, x, act, s, x1, x_split);
        case T_Q6_K: return gateup_dispatch<T_Q6_K>(ex, ids, n_slot, hidden, ffn, x, act, s, x1, x_split);
        case T_IQ2_XS: return gateup_dispatch<T_IQ2_XS>(ex, ids, n_slot, hidden, ffn, x, act, s, x1, x_split);
        case T_IQ1_M: return gateup_dispatch<T_IQ1_M>(ex, ids, n_slot, hidden, ffn, x, act, s, x1, x_split);
        default: return hipErrorInvalidValue;
    }
}

// down projection of the selected experts fused with the weighted sum and the shared expert. A workgroup owns 64 / LPR output
// rows; its four waves split the top_k + 1 matrices between them (slot k goes to wave k % 4, the shared expert is slot top_k), each
// stages only its own slots' activations, and wave 0 adds the four partial sums in a fixed order.
template <uint32_t TD, uint32_t TS, int LPR>
__global__ __launch_bounds__(256) void moe_down_combine_kernel(const uint8_t *base, uint64_t stride, uint64_t down_off,
                                                               const uint32_t *ids, const float *weights, uint32_t top_k,
                                                               const uint8_t *sh_down, const float *scalar,
                                                               uint32_t hidden, uint32_t ffn,
                                                               const float *act, const float *sh_act, float *out,
                                                               const float *resid_a, const float *resid_b, uint32_t id_limit) {
    extern __shared__ float as[];                          // [top_k + 1][padded ffn], then [4][64 / LPR] partial sums
    constexpr uint32_t kRows = 64u / LPR;
    const uint32_t fp = ffn + (ffn >> 5);
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t n_slot = top_k + (sh_down ? 1u : 0u);
    float *partial = as + (size_t)(top_k + 1u) * fp;
    for (uint32_t k = wave; k < n_slot; k += 4u) {
        const float *src = k < top_k ? act + (size_t)k * ffn : sh_act;
        for (uint32_t i = lane; i < ffn; i += 64u) as[k * fp + pad32(i)] = src[i];
    }
    __syncthreads();
    const uint32_t sub = lane % LPR, rl = lane / LPR, r = blockIdx.x * kRows + rl;
    const uint64_t rbd = (uint64_t)(ffn / 256u) * Fmt<TD>::kBlock, rbs = (uint64_t)(ffn / 256u) * Fmt<TS>::kBlock;
    float total = 0.0f;
    for (uint32_t k = wave; k < n_slot; k += 4u) {
        float part = 0.0f;
        if (r < hidden) {
            if (k < top_k) {
                const uint8_t *row = base + (uint64_t)guarded_id(ids[k], id_limit, nullptr) * stride + down_off + (uint64_t)r * rbd;
                for (uint32_t c = sub; c < ffn / 32u; c += LPR) part += chunk_dot<TD>(row, c, as + k * fp + 33u * c);
            } else {
                const uint8_t *row = sh_down + (uint64_t)r * rbs;
                for (uint32_t c = sub; c < ffn / 32u; c += LPR) part += chunk_dot<TS>(row, c, as + k * fp + 33u * c);
            }
        }
        part = sub_reduce<LPR>(part);
        total = fmaf(k < top_k ? weights[k] : scalar[0], part, total);
    }
    if (sub == 0u) partial[wave * kRows + rl] = total;
    __syncthreads();
    if (wave == 0u && sub == 0u && r < hidden) {
        const float sum = (partial[rl] + partial[kRows + rl]) + (partial[2u * kRows + rl] + partial[3u * kRows + rl]);
        out[r] = resid_a ? (resid_a[r] + resid_b[r]) + sum : sum;      // block step: residual added here
    }
}

template <uint32_t TD, uint32_t TS>
static hipError_t down_dispatch(const ExpertSet &ex, const uint32_t *ids, const float *weights, uint32_t top_k,
                                const ExpertSet &sh, const float *scalar, uint32_t hidden, uint32_t ffn,
                                const float *act, const float *sh_act, float *out, hipStream_t s) {
    const uint32_t lpr = lanes_per_row(ffn);
    const dim3 grid((hidden + 64u / lpr - 1u) / (64u / lpr));
    const size_t lds = ((size_t)(top_k + 1u) * padded_floats(ffn) + 4u * (64u / lpr)) * sizeof(float);
    const uint8_t *shd = sh.base ? sh.base + sh.gate_bytes + sh.up_bytes : nullptr;
    const uint64_t off = ex.gate_bytes + ex.up_bytes;
#define REDHIP_DOWN(L) REDHIP_LAUNCH((moe_down_combine_kernel<TD, TS, L>), dim3(grid), dim3(256), lds, s, ex.base, ex.stride, off, ids, weights, top_k, shd, scalar, hidden, ffn, act, sh_act, out, block_context().resid_a, block_context().resid_b, route_guard().id_limit)
    switch (lpr) {
        case 64: REDHIP_DOWN(64); break;
        case 32: REDHIP_DOWN(32); break;
        case 16: REDHIP_DOWN(16); break;
        default: REDHIP_DOWN(8); break;
    }
#undef REDHIP_DOWN
    return hipGetLastError();
}

template <uint32_t TD>
static hipError_t down_dispatch_shared(const ExpertSet &ex, const uint32_t *ids, const float *weights, uint32_t top_k,
                                       const ExpertSet &sh, const float *scalar, uint32_t hidden, uint32_t ffn,
                                       const float *act, const float *sh_act, float *out, hipStream_t s) {
    switch (sh.base ? sh.down_type : (TD == T_IQ2_XS || TD == T_IQ1_M) ? T_IQ2_XXS : TD) {      // without a shared expert TS is never read
        case T_IQ2_XXS: return down_dispatch<TD, T_IQ2_XXS>(ex, ids, weights, top_k, sh, scalar, hidden, ffn, act, sh_act, out, s);
        case T_IQ3_S: return down_dispatch<TD, T_IQ3_S>(ex, ids, weights, top_k, sh, scalar, hidden, ffn, act, sh_act, out, s);
        case T_Q6_K: return down_dispatch<TD, T_Q6_K>(ex, ids, weights, top_k, sh, scalar, hidden, ffn, act, sh_act, out, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_moe_down_combine(const ExpertSet &ex, const uint32_t *ids, const float *weights, uint32_t top_k,
                                   const ExpertSet &shared, const float *scalar, uint32_t hidden, uint32_t ffn,
                                   const float *act, const float *shared_act, float *out, hipStream_t s) {
    hipError_t e = ensure_tables();
    if (e != hipSuccess) return e;
    if (hidden % 256u || ffn % 256u || ((size_t)(top_k + 1u) * padded_floats(ffn) + 32u) * 4u > 64u * 1024u) return hipErrorInvalidValue;
    switch (ex.down_type) {
        case T_IQ2_XXS: return down_dispatch_shared<T_IQ2_XXS>(ex, ids, weights, top_k, shared, scalar, hidden, ffn, act, shared_act, out, s);
        case T_IQ3_S: return down_dispatch_shared<T_IQ3_S>(ex, ids, weights, top_k, shared, scalar, hidden, ffn, act, shared_act, out, s);
        case T_Q6_K: return down_dispatch_shared<T_Q6_K>(ex, ids, weights, top_k, shared, scalar, hidden, ffn, act, shared_act, out, s);
        case T_IQ2_XS: return down_dispatch_shared<T_IQ2_XS>(ex, ids, weights, top_k, shared, scalar, hidden, ffn, act, shared_act, out, s);
        case T_IQ1_M: return down_dispatch_shared<T_IQ1_M>(ex, ids, weights, top_k, shared, scalar, hidden, ffn, act, shared_act, out, s);
        default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------- batched experts over grouped (expert, token) pairs

// Pairs are sorted by expert (expert_start[u] .. expert_start[u+1]); a workgroup takes one expert and a tile of
// rows, decodes every weight once per slice of up to kPairTile pairs and applies it to each pair's activations,
// so an expert's bytes are read once however many tokens selected it. The shared expert runs through the same
// kernels as a single "expert" whose pairs are all the tokens.
constexpr int kPairTile = 8;

struct PairArgs {
    const uint8_t *base;           // expert e at base + e * stride
    uint64_t stride, matrix_off, second_off;      // gate (or down) at matrix_off, up at second_off
    const uint32_t *uid;           // [U] expert of group u, or nullptr: expert 0
    const uint32_t *expert_start;  // [U + 1]
    const uint32_t *pair_token;    // [P] token of each pair, or nullptr: pair p is token p
    const uint32_t *n_unique;      // [1] number of groups, or nullptr: one group
    uint32_t n_pairs_total;        // used when expert_start == nullptr: one group of this many pairs
    const uint64_t *table;         // [U] base address of group u's expert (a slot table), or nullptr: base + e * stride
};

template <uint32_t T, int LPR>
__global__ __launch_bounds__(256) void batch_gateup_kernel(PairArgs a, uint32_t hidden, uint32_t ffn, const float *x, float *act) {
    extern __shared__ float xs[];                                     // [kPairTile][padded hidden]
    const uint32_t u = blockIdx.y;
    if (a.n_unique && u >= a.n_unique[0]) return;
    const uint32_t e = a.uid ? a.uid[u] : 0u;
    const uint32_t p0 = a.expert_start ? a.expert_start[u] : 0u, p1 = a.expert_start ? a.expert_start[u + 1u] : a.n_pairs_total;
    const uint32_t hp = hidden + (hidden >> 5);
    const uint32_t sub = threadIdx.x % LPR, r = blockIdx.x * (256u / LPR) + threadIdx.x / LPR;
    const uint64_t rb = (uint64_t)(hidden / 256u) * Fmt<T>::kBlock;
    const uint8_t *ebase = a.table ? reinterpret_cast<const uint8_t *>(a.table[u]) : a.base + (uint64_t)e * a.stride;
    const uint8_t *grow = ebase + a.matrix_off + (uint64_t)r * rb;
    const uint8_t *urow = ebase + a.second_off + (uint64_t)r * rb;
    for (uint32_t c0 = p0; c0 < p1; c0 += kPairTile) {
        const uint32_t nb = p1 - c0 < (uint32_t)kPairTile ? p1 - c0 : (uint32_t)kPairTile;
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < nb * hidden; i += 256u) {
            const uint32_t pi = i / hidden, col = i % hidden;
            const uint32_t tok = a.pair_token ? a.pair_token[c0 + pi] : c0 + pi;
            xs[pi * hp + pad32(col)] = x[(uint64_t)tok * hidden + col];
        }
        __syncthreads();
        float g[kPairTile], v[kPairTile];
#pragma unroll
        for (int i = 0; i < kPairTile; ++i) { g[i] = 0.0f; v[i] = 0.0f; }
        if (r < ffn) {
            for (uint32_t c = sub; c < hidden / 32u; c += LPR) {
                float wg[32], wu[32];
                decode32<T>(grow, c, wg);
                decode32<T>(urow, c, wu);
#pragma unroll
                for (int i = 0; i < kPairTile; ++i) {
                    if ((uint32_t)i < nb) {
                        const float *xv = xs + i * hp + 33u * c;
                        float sg = 0.0f, su = 0.0f;
#pragma unroll
                        for (int j = 0; j < 32; ++j) { sg = fmaf(wg[j], xv[j], sg); su = fmaf(wu[j], xv[j], su); }
                        g[i] += sg;
                        v[i] += su;
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kPairTile; ++i) {
            if ((uint32_t)i < nb) {
                const float gs = sub_reduce<LPR>(g[i]), us = sub_reduce<LPR>(v[i]);
                if (sub == 0u && r < ffn) act[(uint64_t)(c0 + i) * ffn + r] = silu_mul(gs, us);
            }
        }
    }
}

template <uint32_t T, int LPR>
__global__ __launch_bounds__(256) void batch_down_kernel(PairArgs a, uint32_t hidden, uint32_t ffn, const float *act, float *tmp) {
    extern __shared__ float as[];                                     // [kPairTile][padded ffn]
    const uint32_t u = blockIdx.y;
    if (a.n_unique && u >= a.n_unique[0]) return;
    const uint32_t e = a.uid ? a.uid[u] : 0u;
    const uint32_t p0 = a.expert_start ? a.expert_start[u] : 0u, p1 = a.expert_start ? a.expert_start[u + 1u] : a.n_pairs_total;
    const uint32_t fp = ffn + (ffn >> 5);
    const uint32_t sub = threadIdx.x % LPR, r = blockIdx.x * (256u / LPR) + threadIdx.x / LPR;
    const uint64_t rb = (uint64_t)(ffn / 256u) * Fmt<T>::kBlock;
    const uint8_t *row = (a.table ? reinterpret_cast<const uint8_t *>(a.table[u]) : a.base + (uint64_t)e * a.stride) + a.matrix_off + (uint64_t)r * rb;
    for (uint32_t c0 = p0; c0 < p1; c0 += kPairTile) {
        const uint32_t nb = p1 - c0 < (uint32_t)kPairTile ? p1 - c0 : (uint32_t)kPairTile;
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < nb * ffn; i += 256u) as[(i / ffn) * fp + pad32(i % ffn)] = act[(uint64_t)c0 * ffn + i];
        __syncthreads();
        float s[kPairTile];
#pragma unroll
        for (int i = 0; i < kPairTile; ++i) s[i] = 0.0f;
        if (r < hidden) {
            for (uint32_t c = sub; c < ffn / 32u; c += LPR) {
                float w[32];
                decode32<T>(row, c, w);
#pragma unroll
                for (int i = 0; i < kPairTile; ++i) {
                    if ((uint32_t)i < nb) {
                        const float *av = as + i * fp + 33u * c;
                        float t = 0.0f;
#pragma unroll
                        for (int j = 0; j < 32; ++j) t = fmaf(w[j], av[j], t);
                        s[i] += t;
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kPairTile; ++i) {
            if ((uint32_t)i < nb) {
                const float t = sub_reduce<LPR>(s[i]);
                if (sub == 0u && r < hidden) tmp[(uint64_t)(c0 + i) * hidden + r] = t;
            }
        }
    }
}

// out[t][r] = sum_k pair_weight[p_k] * tmp[p_k][r] (p_k = tok_pair[t][k], selection order) + scalar[t] * sh_tmp[t][r]
// Four rows per thread; a token's pair indices, weights and rows (top_k <= 16) are all requested before the first is used - as a loop
// over k every term was three dependent round trips - and added in selection order as before.
__global__ __launch_bounds__(256) void batch_combine_kernel(const float *tmp, const float *pair_weight, const uint32_t *tok_pair, uint32_t top_k,
                                                            const float *sh_tmp, const float *scalar, uint32_t hidden, float *out,
                                                            const float *resid_a, const float *resid_b) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x, t = blockIdx.y, H4 = hidden / 4u;
    if (c >= H4) return;
    uint32_t p[16];
    float w[16];
    float4 v[16];
#pragma unroll
    for (uint32_t k = 0; k < 16u; ++k) p[k] = k < top_k ? tok_pair[(uint64_t)t * top_k + k] : 0u;
#pragma unroll
    for (uint32_t k = 0; k < 16u; ++k) {
        w[k] = 0.0f;
        v[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (k < top_k) {                                   // (uniform: no row is read for the unused terms)
            w[k] = pair_weight[p[k]];
            v[k] = reinterpret_cast<const float4 *>(tmp)[(uint64_t)p[k] * H4 + c];
        }
    }
    float4 sh = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    const float sc = sh_tmp ? scalar[t] : 0.0f;
    if (sh_tmp) sh = reinterpret_cast<const float4 *>(sh_tmp)[(uint64_t)t * H4 + c];
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
    for (uint32_t k = 0; k < 16u; ++k) {
        if (k < top_k) {
            acc.x = fmaf(w[k], v[k].x, acc.x); acc.y = fmaf(w[k], v[k].y, acc.y);
            acc.z = fmaf(w[k], v[k].z, acc.z); acc.w = fmaf(w[k], v[k].w, acc.w);
        }
    }
    if (sh_tmp) { acc.x = fmaf(sc, sh.x, acc.x); acc.y = fmaf(sc, sh.y, acc.y); acc.z = fmaf(sc, sh.z, acc.z); acc.w = fmaf(sc, sh.w, acc.w); }
    const uint64_t at = (uint64_t)t * H4 + c;
    if (resid_a) {
        const float4 ra = reinterpret_cast<const float4 *>(resid_a)[at], rb = reinterpret_cast<const float4 *>(resid_b)[at];
        acc = make_float4((ra.x + rb.x) + acc.x, (ra.y + rb.y) + acc.y, (ra.z + rb.z) + acc.z, (ra.w + rb.w) + acc.w);
    }
    reinterpret_cast<float4 *>(out)[at] = acc;
}

// the same sum for top_k > 16: blocks of sixteen terms requested together, every term added in selection order
__global__ __launch_bounds__(256) void batch_combine_loop_kernel(const float *tmp, const float *pair_weight, const uint32_t *tok_pair, uint32_t top_k,
                                                                 const float *sh_tmp, const float *scalar, uint32_t hidden, float *out,
                                                                 const float *resid_a, const float *resid_b) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x, t = blockIdx.y, H4 = hidden / 4u;
    if (c >= H4) return;
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (uint32_t k0 = 0; k0 < top_k; k0 += 16u) {
        uint32_t p[16];
        float w[16];
        float4 v[16];
#pragma unroll
        for (uint32_t k = 0; k < 16u; ++k) p[k] = k0 + k < top_k ? tok_pair[(uint64_t)t * top_k + k0 + k] : 0u;
#pragma unroll
        for (uint32_t k = 0; k < 16u; ++k) {
            w[k] = 0.0f;
            v[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (k0 + k < top_k) {
                w[k] = pair_weight[p[k]];
                v[k] = reinterpret_cast<const float4 *>(tmp)[(uint64_t)p[k] * H4 + c];
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < 16u; ++k) {
            if (k0 + k < top_k) {
                acc.x = fmaf(w[k], v[k].x, acc.x); acc.y = fmaf(w[k], v[k].y, acc.y);
                acc.z = fmaf(w[k], v[k].z, acc.z); acc.w = fmaf(w[k], v[k].w, acc.w);
            }
        }
    }
    if (sh_tmp) {
        const float sc = scalar[t];
        const float4 sh = reinterpret_cast<const float4 *>(sh_tmp)[(uint64_t)t * H4 + c];
        acc.x = fmaf(sc, sh.x, acc.x); acc.y = fmaf(sc, sh.y, acc.y); acc.z = fmaf(sc, sh.z, acc.z); acc.w = fmaf(sc, sh.w, acc.w);
    }
    const uint64_t at = (uint64_t)t * H4 + c;
    if (resid_a) {
        const float4 ra = reinterpret_cast<const float4 *>(resid_a)[at], rb = reinterpret_cast<const float4 *>(resid_b)[at];
        acc = make_float4((ra.x + rb.x) + acc.x, (ra.y + rb.y) + acc.y, (ra.z + rb.z) + acc.z, (ra.w + rb.w) + acc.w);
    }
    reinterpret_cast<float4 *>(out)[at] = acc;
}

template <uint32_t T>
static hipError_t batch_gateup_dispatch(const PairArgs &a, uint32_t n_groups, uint32_t hidden, uint32_t ffn, const float *x, float *act, hipStream_t s) {
    const uint32_t lpr = lanes_per_row(hidden);
    const dim3 grid((ffn + 256u / lpr - 1u) / (256u / lpr), n_groups);
    const size_t lds = (size_t)kPairTile * padded_floats(hidden) * sizeof(float);
#define REDHIP_BGU(L)                                                                                                              \
    do {                                                                                                                           \
        static bool attr = false;                                                                                                  \
        if (!attr) {                                                                                                               \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(batch_gateup_kernel<T, L>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (e != hipSuccess) return e;                                                                                         \
            attr = true;                                                                                                           \
        }                                                                                                                          \
        REDHIP_LAUNCH((batch_gateup_kernel<T, L>), grid, dim3(256), lds, s, a, hidden, ffn, x, act);                               \
    } while (0)
    switch (lpr) {
        case 64: REDHIP_BGU(64); break;
        case 32: REDHIP_BGU(32); break;
        case 16: REDHIP_BGU(16); break;
        default: REDHIP_BGU(8); break;
    }
#undef REDHIP_BGU
    return hipGetLastError();
}

template <uint32_t T>
static hipError_t batch_down_dispatch(const PairArgs &a, uint32_t n_groups, uint32_t hidden, uint32_t ffn, const float *act, float *tmp, hipStream_t s) {
    const uint32_t lpr = lanes_per_row(ffn);
    const dim3 grid((hidden + 256u / lpr - 1u) / (256u / lpr), n_groups);
    const size_t lds = (size_t)kPairTile * padded_floats(ffn) * sizeof(float);
#define REDHIP_BDN(L)                                                                                                              \
    do {                                                                                                                           \
        static bool attr = false;                                                                                                  \
        if (!attr) {      /* (the default limit is 64 KB: ffn >= 2048 needs more) */                                               \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(batch_down_kernel<T, L>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (e != hipSuccess) return e;                                                                                         \
            attr = true;                                                                                                           \
        }                                                                                                                          \
        REDHIP_LAUNCH((batch_down_kernel<T, L>), grid, dim3(256), lds, s, a, hidden, ffn, act, tmp);                               \
    } while (0)
    switch (lpr) {
        case 64: REDHIP_BDN(64); break;
        case 32: REDHIP_BDN(32); break;
        case 16: REDHIP_BDN(16); break;
        default: REDHIP_BDN(8); break;
    }
#undef REDHIP_BDN
    return hipGetLastError();
}

hipError_t launch_batch_gateup(const ExpertSet &ex, const uint32_t *uid, const uint32_t *expert_start, const uint32_t *pair_token,
                               const uint32_t *n_unique, uint32_t n_groups, uint32_t n_pairs_total, uint32_t hidden, uint32_t ffn,
                               const float *x, float *act, hipStream_t s) {
    if (!n_groups || hidden % 256u || ffn % 256u || (size_t)kPairTile * padded_floats(hidden) * 4u > 160u * 1024u || n_groups > 65535u) return hipErrorInvalidValue;
    const PairArgs a{ex.base, ex.stride, 0u, ex.gate_bytes, uid, expert_start, pair_token, n_unique, n_pairs_total, ex.table};
    switch (ex.gate_up_type) {
        case T_IQ2_XXS: return batch_gateup_dispatch<T_IQ2_XXS>(a, n_groups, hidden, ffn, x, act, s);
        case T_IQ3_S: return batch_gateup_dispatch<T_IQ3_S>(a, n_groups, hidden, ffn, x, act, s);
        case T_Q6_K: return batch_gateup_dispatch<T_Q6_K>(a, n_groups, hidden, ffn, x, act, s);
        case T_IQ2_XS: return batch_gateup_dispatch<T_IQ2_XS>(a, n_groups, hidden, ffn, x, act, s);
        case T_IQ1_M: return batch_gateup_dispatch<T_IQ1_M>(a, n_groups, hidden, ffn, x, act, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_batch_down(const ExpertSet &ex, const uint32_t *uid, const uint32_t *expert_start, const uint32_t *n_unique,
                             uint32_t n_groups, uint32_t n_pairs_total, uint32_t hidden, uint32_t ffn, const float *act, float *tmp, hipStream_t s) {
    if (!n_groups || hidden % 256u || ffn % 256u || (size_t)kPairTile * padded_floats(ffn) * 4u > 160u * 1024u || n_groups > 65535u) return hipErrorInvalidValue;
    const PairArgs a{ex.base, ex.stride, ex.gate_bytes + ex.up_bytes, 0u, uid, expert_start, nullptr, n_unique, n_pairs_total, ex.table};
    switch (ex.down_type) {
        case T_IQ2_XXS: return batch_down_dispatch<T_IQ2_XXS>(a, n_groups, hidden, ffn, act, tmp, s);
        case T_IQ3_S: return batch_down_dispatch<T_IQ3_S>(a, n_groups, hidden, ffn, act, tmp, s);
        case T_Q6_K: return batch_down_dispatch<T_Q6_K>(a, n_groups, hidden, ffn, act, tmp, s);
        case T_IQ2_XS: return batch_down_dispatch<T_IQ2_XS>(a, n_groups, hidden, ffn, act, tmp, s);
        case T_IQ1_M: return batch_down_dispatch<T_IQ1_M>(a, n_groups, hidden, ffn, act, tmp, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_batch_combine(const float *tmp, const float *pair_weight, const uint32_t *tok_pair, uint32_t ntok, uint32_t top_k,
                                const float *sh_tmp, const float *scalar, uint32_t hidden, float *out, hipStream_t s) {
    if (hidden % 4u || !top_k) return hipErrorInvalidValue;
    const dim3 grid((hidden / 4u + 255u) / 256u, ntok);
    if (top_k <= 16u) REDHIP_LAUNCH(batch_combine_kernel, grid, dim3(256), 0, s, tmp, pair_weight, tok_pair, top_k, sh_tmp, scalar, hidden, out, block_context().resid_a, block_context().resid_b);
    else REDHIP_LAUNCH(batch_combine_loop_kernel, grid, dim3(256), 0, s, tmp, pair_weight, tok_pair, top_k, sh_tmp, scalar, hidden, out, block_context().resid_a, block_context().resid_b);
    return hipGetLastError();
}

// out[i] = sum_k weights[k] * tmp[k][row_start + i], experts accumulated in the order of the list
__global__ __launch_bounds__(256) void weighted_sum_kernel(const float *tmp, const float *weights, uint32_t top_k, uint32_t hidden,
                                                           uint32_t row_start, uint32_t row_count, float *out) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= row_count) return;
    float acc = 0.0f;
    for (uint32_t k0 = 0; k0 < top_k; k0 += 16u) {      // sixteen terms requested together, added in the order of the list
        float w[16], v[16];
#pragma unroll
        for (uint32_t k = 0; k < 16u; ++k) {
            w[k] = 0.0f;
            v[k] = 0.0f;
            if (k0 + k < top_k) { w[k] = weights[k0 + k]; v[k] = tmp[(uint64_t)(k0 + k) * hidden + row_start + i]; }
        }
#pragma unroll
        for (uint32_t k = 0; k < 16u; ++k) if (k0 + k < top_k) acc = fmaf(w[k], v[k], acc);
    }
    out[i] = acc;
}

hipError_t launch_weighted_sum(const float *tmp, const float *weights, uint32_t top_k, uint32_t hidden, uint32_t row_start,
                               uint32_t row_count, float *out, hipStream_t s) {
    if (!top_k || !row_count || row_start >= hidden || row_count > hidden - row_start) return hipErrorInvalidValue;
    REDHIP_LAUNCH(weighted_sum_kernel, dim3((row_count + 255u) / 256u), dim3(256), 0, s, tmp, weights, top_k, hidden, row_start, row_count, out);
    return hipGetLastError();
}

// ---------------------------------------------------------------- token grouping (pair sort)

// exclusive prefix sum over the 1024 threads of a workgroup (16 waves): in-wave shuffles, then the 16 wave totals
__device__ __forceinline__ uint32_t block_scan_1024(uint32_t v, uint32_t *wave_tot /* [17] */, uint32_t &total) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { const uint32_t n = __shfl_up(inc, o, 64); if (lane >= (uint32_t)o) inc += n; }
    if (lane == 63u) wave_tot[wave] = inc;
    __syncthreads();
    if (threadIdx.x == 0u) {
        uint32_t acc = 0u;
#pragma unroll
        for (int w = 0; w < 16; ++w) { const uint32_t t = wave_tot[w]; wave_tot[w] = acc; acc += t; }
        wave_tot[16] = acc;
    }
    __syncthreads();
    total = wave_tot[16];
    const uint32_t ex = wave_tot[wave] + inc - v;
    __syncthreads();                               // wave_tot may be reused right away
    return ex;
}

// One workgroup. For every (token, k) pair p = t * top_k + k:
//   first[e]   = smallest p that names expert e            -> experts numbered in first-appearance order
//   member[e]  = bitmap over tokens that selected e        -> rank of a pair inside its expert = popcount below t
// which gives the stable counting sort of the host loop it replaces without a serial pass. All of it runs on one
// compute unit, so the instruction count is what it costs: the token of a pair comes from a multiply-high by
// ceil(2^32 / top_k) (exact while pairs * top_k < 2^32), and with PREFIX the bit counts of the words below a token's word come
// from a table made once per expert (which also yields the expert's pair count) instead of a loop per pair.
template <bool PREFIX>
__global__ __launch_bounds__(1024) void group_pairs_kernel(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t top_k_magic,
                                                           uint32_t n_expert, uint32_t *uid, uint32_t *expert_start,
                                                           uint32_t *pair_token, float *pair_weight, uint32_t *tok_pair,
                                                           uint32_t *n_unique, uint32_t *status, uint32_t cache_ids, TileLists tiles) {
    extern __shared__ uint32_t sm[];
    __shared__ uint32_t tile_tot[3][16];
    const uint32_t words = (ntok + 31u) / 32u, P = ntok * top_k, tid = threadIdx.x;
    uint32_t *first = sm;                          // [n_expert]
    uint32_t *count = first + n_expert;            // [n_expert]
    uint32_t *dense = count + n_expert;            // [n_expert]
    uint32_t *start = dense + n_expert;            // [n_expert + 1] by dense index
    uint32_t *uid_l = start + n_expert + 1u;       // [1024] experts by dense index (n_expert <= 1024)
    uint32_t *wave_tot = uid_l + 1024u;            // [17]
    uint32_t *member = wave_tot + 17u;             // [n_expert][words]
    uint32_t *below = member + n_expert * words;   // [n_expert][words] when PREFIX: members in the words before this one
    uint32_t *ids_l = cache_ids ? below + (PREFIX ? n_expert * words : 0u) : nullptr;      // [P] the clamped ids, when LDS has room: the later passes need no second trip to device memory
    auto token_of = [&](uint32_t p) { return top_k == 1u ? p : __umulhi(p, top_k_magic); };
    // the ids are the caller's: clamped into the tables (reported once, in the first pass)
    auto id_of = [&](uint32_t p) { if (ids_l) return ids_l[p]; const uint32_t e = ids[p]; return e < n_expert ? e : n_expert - 1u; };
    // Up to eight pairs per thread (chunks of up to 8192 pairs) are requested here, ids and weights, before anything else: read inside the
    // passes below, each would be a round trip of its own (the stores of the last pass keep the loads of the next pair behind them).
    constexpr uint32_t kRegPairs = 8u;
    const bool in_regs = P <= kRegPairs * 1024u;
    uint32_t ereg[kRegPairs];
    float wreg[kRegPairs];
    if (in_regs) {
#pragma unroll
        for (uint32_t j = 0; j < kRegPairs; ++j) {
            const uint32_t p = tid + 1024u * j;
            ereg[j] = p < P ? ids[p] : 0u;
            wreg[j] = p < P ? weights[p] : 0.0f;
        }
    }
    for (uint32_t i = tid; i < n_expert; i += 1024u) { first[i] = 0xffffffffu; count[i] = 0u; dense[i] = 0u; }
    for (uint32_t i = tid; i < n_expert * words; i += 1024u) member[i] = 0u;
    __syncthreads();
    auto enter = [&](uint32_t p, uint32_t raw) {
        const uint32_t e = guarded_id(raw, n_expert, status), t = token_of(p);
        if (ids_l) ids_l[p] = e;
        atomicMin(&first[e], p);
        if constexpr (!PREFIX) atomicAdd(&count[e], 1u);
        if ((atomicOr(&member[e * words + (t >> 5)], 1u << (t & 31u)) & (1u << (t & 31u))) && status) atomicOr(status, 2u);      // the token names this expert twice
        return e;
    };
    if (in_regs) {
#pragma unroll
        for (uint32_t j = 0; j < kRegPairs; ++j) { const uint32_t p = tid + 1024u * j; if (p < P) ereg[j] = enter(p, ereg[j]); }
    } else {
        for (uint32_t p = tid; p < P; p += 1024u) enter(p, ids[p]);
    }
    __syncthreads();
    if constexpr (PREFIX) {
        for (uint32_t e = tid; e < n_expert; e += 1024u) {
            uint32_t run = 0u;
            for (uint32_t w = 0; w < words; ++w) { below[e * words + w] = run; run += __popc(member[e * words + w]); }
            count[e] = run;
        }
    }
    // exclusive scan of "pair p is the first appearance of its expert", P elements in per-thread runs
    const uint32_t per = (P + 1023u) / 1024u;
    uint32_t mine = 0u;
    for (uint32_t j = 0; j < per; ++j) { const uint32_t p = tid * per + j; if (p < P && first[id_of(p)] == p) ++mine; }
    uint32_t U = 0u;
    uint32_t run = block_scan_1024(mine, wave_tot, U);
    for (uint32_t j = 0; j < per; ++j) {
        const uint32_t p = tid * per + j;
        if (p < P && first[id_of(p)] == p) { const uint32_t e = id_of(p); dense[e] = run; uid_l[run] = e; uid[run] = e; ++run; }
    }
    __syncthreads();
    // exclusive scan of the per-expert pair counts in dense order (U <= n_expert <= 1024: one per thread)
    uint32_t all = 0u;
    const uint32_t my_start = block_scan_1024(tid < U ? count[uid_l[tid]] : 0u, wave_tot, all);
    if (tid < U) { start[tid] = my_start; expert_start[tid] = my_start; }
    if (tid == 0u) { start[U] = all; expert_start[U] = all; n_unique[0] = U; }
    __syncthreads();
    auto place = [&](uint32_t p, uint32_t e, float wt) {
        const uint32_t t = token_of(p);
        const uint32_t *bits = member + e * words;
        uint32_t rank = __popc(bits[t >> 5] & ((1u << (t & 31u)) - 1u));
        if constexpr (PREFIX) rank += below[e * words + (t >> 5)];
        else for (uint32_t w = 0; w < (t >> 5); ++w) rank += __popc(bits[w]);
        const uint32_t pos = start[dense[e]] + rank;
        pair_token[pos] = t;
        pair_weight[pos] = wt;
        tok_pair[p] = pos;
    };
    if (in_regs) {
#pragma unroll
        for (uint32_t j = 0; j < kRegPairs; ++j) { const uint32_t p = tid + 1024u * j; if (p < P) place(p, ereg[j], wreg[j]); }
    } else {
        for (uint32_t p = tid; p < P; p += 1024u) place(p, id_of(p), weights[p]);
    }
    // the tile lists of the prefill kernels, from the group starts still in LDS: no launch of their own
    if (tiles.tile_group) build_tile_lists(U, tid < U ? start[tid] : 0u, tid < U ? start[tid + 1u] - start[tid] : 0u, P, tiles, tile_tot);
}

// The same sort for chunks of more than 512 tokens, whose token bitmaps per expert would not fit the LDS (2048 tokens x 512 experts: 128
// KB, and as much again for the prefix counts - without them a pair's rank is a loop over up to 64 words, 300 us per chunk): the first
// appearances and the pair counts of the experts come from one pass over all pairs, then the pairs are placed block by block of 512
// tokens - bitmaps and prefix counts of one block (32 KB each), a cursor per expert that advances by the block's count. Same outputs in
// the same (stable) order; one workgroup, the time grows with the number of blocks.
constexpr uint32_t kGroupBlockTokens = 512u, kGroupBlockWords = kGroupBlockTokens / 32u;
__global__ __launch_bounds__(1024) void group_pairs_blocked_kernel(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t top_k_magic,
                                                                   uint32_t n_expert, uint32_t *uid, uint32_t *expert_start,
                                                                   uint32_t *pair_token, float *pair_weight, uint32_t *tok_pair,
                                                                   uint32_t *n_unique, uint32_t *status, uint32_t cache_ids, TileLists tiles) {
    extern __shared__ uint32_t sm[];
    __shared__ uint32_t tile_tot[3][16];
    constexpr uint32_t WB = kGroupBlockWords;
    const uint32_t P = ntok * top_k, tid = threadIdx.x;
    uint32_t *first = sm;                          // [n_expert]
    uint32_t *count = first + n_expert;            // [n_expert]
    uint32_t *dense = count + n_expert;            // [n_expert]
    uint32_t *cursor = dense + n_expert;           // [n_expert] pairs of the expert placed by the blocks before
    uint32_t *start = cursor + n_expert;           // [n_expert + 1] by dense index
    uint32_t *uid_l = start + n_expert + 1u;       // [1024]
    uint32_t *wave_tot = uid_l + 1024u;            // [17]
    uint32_t *member = wave_tot + 17u;             // [n_expert][WB] tokens of the block that selected the expert
    uint32_t *below = member + n_expert * WB;      // [n_expert][WB] members in the words before this one
    uint32_t *ids_l = cache_ids ? below + n_expert * WB : nullptr;      // [P] the clamped ids
    auto token_of = [&](uint32_t p) { return top_k == 1u ? p : __umulhi(p, top_k_magic); };
    auto id_of = [&](uint32_t p) { if (ids_l) return ids_l[p]; const uint32_t e = ids[p]; return e < n_expert ? e : n_expert - 1u; };
    for (uint32_t i = tid; i < n_expert; i += 1024u) { first[i] = 0xffffffffu; count[i] = 0u; dense[i] = 0u; cursor[i] = 0u; }
    __syncthreads();
    for (uint32_t pb = tid; pb < P; pb += 8u * 1024u) {      // eight ids per thread requested together
        uint32_t raw[8];
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) { const uint32_t p = pb + 1024u * j; raw[j] = p < P ? ids[p] : 0u; }
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) {
            const uint32_t p = pb + 1024u * j;
            if (p < P) {
                const uint32_t e = guarded_id(raw[j], n_expert, status);
                if (ids_l) ids_l[p] = e;
                atomicMin(&first[e], p);
                atomicAdd(&count[e], 1u);
            }
        }
    }
    __syncthreads();
    // experts numbered in first-appearance order: exclusive scan of "pair p is the first appearance of its expert" in per-thread runs
    const uint32_t per = (P + 1023u) / 1024u;
    uint32_t mine = 0u;
    for (uint32_t j = 0; j < per; ++j) { const uint32_t p = tid * per + j; if (p < P && first[id_of(p)] == p) ++mine; }
    uint32_t U = 0u;
    uint32_t run = block_scan_1024(mine, wave_tot, U);
    for (uint32_t j = 0; j < per; ++j) {
        const uint32_t p = tid * per + j;
        if (p < P && first[id_of(p)] == p) { const uint32_t e = id_of(p); dense[e] = run; uid_l[run] = e; uid[run] = e; ++run; }
    }
    __syncthreads();
    uint32_t all = 0u;
    const uint32_t my_start = block_scan_1024(tid < U ? count[uid_l[tid]] : 0u, wave_tot, all);
    if (tid < U) { start[tid] = my_start; expert_start[tid] = my_start; }
    if (tid == 0u) { start[U] = all; expert_start[U] = all; n_unique[0] = U; }
    __syncthreads();
    for (uint32_t t0 = 0; t0 < ntok; t0 += kGroupBlockTokens) {
        const uint32_t t1 = t0 + kGroupBlockTokens < ntok ? t0 + kGroupBlockTokens : ntok, p0 = t0 * top_k, p1 = t1 * top_k;
        // the block's weights (at most 512 x 16 pairs: eight per thread) are requested here and stored behind the bitmap passes
        float wreg[8];
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) { const uint32_t p = p0 + tid + 1024u * j; wreg[j] = p < p1 ? weights[p] : 0.0f; }
        for (uint32_t i = tid; i < n_expert * WB; i += 1024u) member[i] = 0u;
        __syncthreads();
        for (uint32_t p = p0 + tid; p < p1; p += 1024u) {
            const uint32_t e = id_of(p), t = token_of(p) - t0, bit = 1u << (t & 31u);
            if ((atomicOr(&member[e * WB + (t >> 5)], bit) & bit) && status) atomicOr(status, 2u);      // the token names this expert twice
        }
        __syncthreads();
        uint32_t block_count = 0u;                     // of expert tid (n_expert <= 1024)
        if (tid < n_expert) {
#pragma unroll
            for (uint32_t w = 0; w < WB; ++w) { below[tid * WB + w] = block_count; block_count += __popc(member[tid * WB + w]); }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) {
            const uint32_t p = p0 + tid + 1024u * j;
            if (p < p1) {
                const uint32_t e = id_of(p), tok = token_of(p), t = tok - t0;
                const uint32_t rank = below[e * WB + (t >> 5)] + __popc(member[e * WB + (t >> 5)] & ((1u << (t & 31u)) - 1u));
                const uint32_t pos = start[dense[e]] + cursor[e] + rank;
                pair_token[pos] = tok;
                pair_weight[pos] = wreg[j];
                tok_pair[p] = pos;
            }
        }
        __syncthreads();
        if (tid < n_expert) cursor[tid] += block_count;
    }
    __syncthreads();
    if (tiles.tile_group) build_tile_lists(U, tid < U ? start[tid] : 0u, tid < U ? start[tid + 1u] - start[tid] : 0u, P, tiles, tile_tot);
}

// ---- the same sort by many workgroups, for large chunks: spans of kGroupSpan tokens, three launches
//   group_count_kernel  one workgroup per span: pairs per expert of the span, and the first pair of every expert (a maximum over ~p, so
//                       that the all-zero scratch means "no pair yet")
//   group_plan_kernel   one workgroup: experts in first-appearance order, their starts, every span's offset inside its expert, the tile
//                       lists; leaves first_key zero for the next chunk
//   group_place_kernel  one workgroup per span: a pair's place = its expert's start + the pairs of the spans before + the tokens of this
//                       span before it that chose the expert (bitmap of the span's tokens per expert in LDS)
// Same outputs in the same stable order as the single-workgroup kernels.
__global__ __launch_bounds__(256) void group_count_kernel(const uint32_t *ids, uint32_t ntok, uint32_t top_k, uint32_t n_expert, GroupScratch gs, uint32_t *status) {
    __shared__ uint32_t hist[1024], key[1024];
    const uint32_t tid = threadIdx.x, b = blockIdx.x;
    const uint32_t t0 = b * kGroupSpan, t1 = t0 + kGroupSpan < ntok ? t0 + kGroupSpan : ntok, p0 = t0 * top_k, p1 = t1 * top_k;
    for (uint32_t e = tid; e < n_expert; e += 256u) { hist[e] = 0u; key[e] = 0u; }
    __syncthreads();
    for (uint32_t p = p0 + tid; p < p1; p += 256u) {
        const uint32_t e = guarded_id(ids[p], n_expert, status);
        atomicAdd(&hist[e], 1u);
        atomicMax(&key[e], ~p);
    }
    __syncthreads();
    for (uint32_t e = tid; e < n_expert; e += 256u) {
        gs.count_blk[(uint64_t)b * n_expert + e] = hist[e];
        if (key[e]) atomicMax(&gs.first_key[e], key[e]);
    }
}

__global__ __launch_bounds__(1024) void group_plan_kernel(GroupScratch gs, uint32_t nb, uint32_t n_expert, uint32_t P, uint32_t *uid, uint32_t *expert_start,
                                                          uint32_t *n_unique, TileLists tiles) {
    __shared__ uint32_t key_l[1024], cnt[1024], uid_l[1024], start[1025], wave_tot[17];
    __shared__ uint32_t tile_tot[3][16];
    const uint32_t tid = threadIdx.x;
    uint32_t my_key = 0u, total = 0u;
    if (tid < n_expert) {
        my_key = gs.first_key[tid];
        gs.first_key[tid] = 0u;                            // ready for the next chunk
        for (uint32_t b0 = 0; b0 < nb; b0 += 16u) {      // sixteen spans' counts requested together, then their running sums stored
            uint32_t c[16];
#pragma unroll
            for (uint32_t i = 0; i < 16u; ++i) c[i] = b0 + i < nb ? gs.count_blk[(uint64_t)(b0 + i) * n_expert + tid] : 0u;
#pragma unroll
            for (uint32_t i = 0; i < 16u; ++i) {
                if (b0 + i < nb) gs.blk_off[(uint64_t)(b0 + i) * n_expert + tid] = total;
                total += c[i];
            }
        }
    }
    key_l[tid] = my_key;
    cnt[tid] = total;
    __syncthreads();
    // first-appearance order: the experts with an earlier first pair (a larger key) come before this one
    uint32_t d = 0u;
    if (my_key) for (uint32_t e = 0; e < n_expert; ++e) d += key_l[e] > my_key ? 1u : 0u;
    uint32_t U = 0u;
    (void)block_scan_1024(my_key ? 1u : 0u, wave_tot, U);
    if (my_key) { uid_l[d] = tid; uid[d] = tid; }
    __syncthreads();
    uint32_t all = 0u;
    const uint32_t my_start = block_scan_1024(tid < U ? cnt[uid_l[tid]] : 0u, wave_tot, all);
    if (tid < U) { start[tid] = my_start; expert_start[tid] = my_start; gs.expert_base[uid_l[tid]] = my_start; }
    if (tid == 0u) { start[U] = all; expert_start[U] = all; n_unique[0] = U; }
    __syncthreads();
    if (tiles.tile_group) build_tile_lists(U, tid < U ? start[tid] : 0u, tid < U ? start[tid + 1u] - start[tid] : 0u, P, tiles, tile_tot);
}

__global__ __launch_bounds__(256) void group_place_kernel(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t top_k_magic,
                                                          uint32_t n_expert, GroupScratch gs, uint32_t *pair_token, float *pair_weight, uint32_t *tok_pair,
                                                          uint32_t *status) {
    constexpr uint32_t W = kGroupSpan / 32u;
    __shared__ uint32_t member[1024 * W];
    const uint32_t tid = threadIdx.x, b = blockIdx.x;
    const uint32_t t0 = b * kGroupSpan, t1 = t0 + kGroupSpan < ntok ? t0 + kGroupSpan : ntok, p0 = t0 * top_k, p1 = t1 * top_k;
    auto token_of = [&](uint32_t p) { return top_k == 1u ? p : __umulhi(p, top_k_magic); };
    // at most kGroupSpan x 16 pairs per span: four per thread, ids and weights requested up front
    uint32_t ereg[4];
    float wreg[4];
#pragma unroll
    for (uint32_t j = 0; j < 4u; ++j) {
        const uint32_t p = p0 + tid + 256u * j;
        const uint32_t e = p < p1 ? ids[p] : 0u;
        ereg[j] = e < n_expert ? e : n_expert - 1u;        // (reported by the counting launch)
        wreg[j] = p < p1 ? weights[p] : 0.0f;
    }
    for (uint32_t i = tid; i < n_expert * W; i += 256u) member[i] = 0u;
    __syncthreads();
#pragma unroll
    for (uint32_t j = 0; j < 4u; ++j) {
        const uint32_t p = p0 + tid + 256u * j;
        if (p < p1) {
            const uint32_t t = token_of(p) - t0, bit = 1u << (t & 31u);
            if ((atomicOr(&member[ereg[j] * W + (t >> 5)], bit) & bit) && status) atomicOr(status, 2u);      // the token names this expert twice
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t j = 0; j < 4u; ++j) {
        const uint32_t p = p0 + tid + 256u * j;
        if (p < p1) {
            const uint32_t e = ereg[j], tok = token_of(p), t = tok - t0;
            uint32_t rank = __popc(member[e * W + (t >> 5)] & ((1u << (t & 31u)) - 1u));
            for (uint32_t w = 0; w < (t >> 5); ++w) rank += __popc(member[e * W + w]);
            const uint32_t pos = gs.expert_base[e] + gs.blk_off[(uint64_t)b * n_expert + e] + rank;
            pair_token[pos] = tok;
            pair_weight[pos] = wreg[j];
            tok_pair[p] = pos;
        }
    }
}

hipError_t launch_group_pairs(const uint32_t *ids, const float *weights, uint32_t ntok, uint32_t top_k, uint32_t n_expert,
                              uint32_t *uid, uint32_t *expert_start, uint32_t *pair_token, float *pair_weight,
                              uint32_t *tok_pair, uint32_t *n_unique, hipStream_t s, const TileLists *tiles, const GroupScratch *scratch) {
    if (!ntok || !top_k || !n_expert || n_expert > 1024u || (uint64_t)ntok * top_k * top_k >= (1ull << 32)) return hipErrorInvalidValue;
    const TileLists tl = tiles ? *tiles : TileLists{};
    const uint32_t words = (ntok + 31u) / 32u;
    const size_t lds = sizeof(uint32_t) * ((size_t)4u * n_expert + 1u + 1024u + 17u + (size_t)n_expert * words);
    constexpr size_t kGroupDynLds = 159u * 1024u;      // (the kernel has a little static LDS beside it)
    const size_t lds_prefix = lds + sizeof(uint32_t) * (size_t)n_expert * words;
    const uint32_t magic = (uint32_t)(((1ull << 32) + top_k - 1u) / top_k);      // top_k == 1 needs none (and would not fit)
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(group_pairs_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGroupDynLds);
        if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void *>(group_pairs_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGroupDynLds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    if (scratch && ntok > kGroupBlockTokens && (ntok + kGroupSpan - 1u) / kGroupSpan <= scratch->blocks && top_k <= 16u) {      // many workgroups, three launches
        const uint32_t nb = (ntok + kGroupSpan - 1u) / kGroupSpan;
        REDHIP_LAUNCH(group_count_kernel, dim3(nb), dim3(256), 0, s, ids, ntok, top_k, n_expert, *scratch, route_guard().status);
        REDHIP_LAUNCH(group_plan_kernel, dim3(1), dim3(1024), 0, s, *scratch, nb, n_expert, ntok * top_k, uid, expert_start, n_unique, tl);
        REDHIP_LAUNCH(group_place_kernel, dim3(nb), dim3(256), 0, s, ids, weights, ntok, top_k, magic, n_expert, *scratch, pair_token, pair_weight, tok_pair,
                      route_guard().status);
        return hipGetLastError();
    }
    const size_t ids_bytes = sizeof(uint32_t) * (size_t)ntok * top_k;
    const size_t lds_blocked = sizeof(uint32_t) * ((size_t)5u * n_expert + 1u + 1024u + 17u + (size_t)2u * n_expert * kGroupBlockWords);
    if (ntok > kGroupBlockTokens && lds_blocked <= kGroupDynLds) {       // larger chunks: block by block
        static bool blocked_attr = false;
        if (!blocked_attr) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(group_pairs_blocked_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGroupDynLds);
            if (e != hipSuccess) return e;
            blocked_attr = true;
        }
        const bool cache = lds_blocked + ids_bytes <= kGroupDynLds;
        REDHIP_LAUNCH(group_pairs_blocked_kernel, dim3(1), dim3(1024), lds_blocked + (cache ? ids_bytes : 0u), s, ids, weights, ntok, top_k, magic, n_expert, uid, expert_start,
                      pair_token, pair_weight, tok_pair, n_unique, route_guard().status, cache ? 1u : 0u, tl);
        return hipGetLastError();
    }
    if (lds > kGroupDynLds) return hipErrorInvalidValue;
    if (lds_prefix <= kGroupDynLds) {
        const bool cache = lds_prefix + ids_bytes <= kGroupDynLds;
        REDHIP_LAUNCH(group_pairs_kernel<true>, dim3(1), dim3(1024), lds_prefix + (cache ? ids_bytes : 0u), s, ids, weights, ntok, top_k, magic, n_expert, uid, expert_start, pair_token,
                      pair_weight, tok_pair, n_unique, route_guard().status, cache ? 1u : 0u, tl);
    } else {
        const bool cache = lds + ids_bytes <= kGroupDynLds;
        REDHIP_LAUNCH(group_pairs_kernel<false>, dim3(1), dim3(1024), lds + (cache ? ids_bytes : 0u), s, ids, weights, ntok, top_k, magic, n_expert, uid, expert_start, pair_token,
                      pair_weight, tok_pair, n_unique, route_guard().status, cache ? 1u : 0u, tl);
    }
    return hipGetLastError();
}

}  // namespace redhip
