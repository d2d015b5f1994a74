// LayerNorm and RMSNorm, forward and backward, for gfx950.
//
// x: [rows, cols]; every row is normalised on its own. A row is cut into
// 16-byte chunks; chunk c = (k * W + w) * L + l belongs to lane l of a group
// of L lanes (a power of two up to 64; several rows share a wave when the
// row is short), register slot k < K and wave w < W of the row's workgroup.
// The row stays in registers (packed, as loaded) between the statistics and
// the output pass, so every element is read from memory once.
//
// Statistics and arithmetic are fp32 whatever the storage type; the mean is
// subtracted before the squares are summed (two passes over registers).
// Results are rounded once to the storage type. gamma / beta (scale /
// offset) are fp32 or of the storage type.
//
// The backward kernel walks over row blocks with a bounded grid, keeps the
// per-column sums for the parameter gradients in registers and writes one
// partial row per workgroup; a second kernel adds the partial rows in a fixed
// order, so results are reproducible from run to run.

#include "common.hpp"
#include "colsum.hpp"

#include <mutex>

namespace nhp {

constexpr int kNormBlockWaves = 4;  // waves per workgroup when a wave holds whole rows
constexpr int kNormScalarThreads = 256;

// Sum over groups of L consecutive lanes (L a power of two, uniform over the wave).
__device__ __forceinline__ float lanes_sum(float v, uint32_t L)
{
    if (L >= 2) v += dpp_move<0xB1>(v);
    if (L >= 4) v += dpp_move<0x4E>(v);
    if (L >= 8) v += dpp_move<0x141>(v);
    if (L >= 16) v += dpp_move<0x140>(v);
    if (L >= 32) v += bitcast<float>(__builtin_amdgcn_ds_swizzle(bitcast<int>(v), 0x401F));
    if (L >= 64) {
        const float a = bitcast<float>(__builtin_amdgcn_readlane(bitcast<int>(v), 0));
        const float b = bitcast<float>(__builtin_amdgcn_readlane(bitcast<int>(v), 32));
        v = a + b;
    }
    return v;
}

// Sum over the W waves of a row group. `slots`: W floats of LDS per row group (the caller
// passes the group's own), not used by another reduction that could still be in flight.
template <int W>
__device__ __forceinline__ float waves_sum(float v, float* slots, int w, int lane)
{
    if constexpr (W == 1) {
        return v;
    } else {
        if (lane == 0) slots[w] = v;
        __syncthreads();
        float r = slots[0];
#pragma unroll
        for (int i = 1; i < W; ++i) r += slots[i];
        return r;
    }
}

// V consecutive parameter values starting at element e (a multiple of V).
template <int DT>
__device__ __forceinline__ void load_params(const void* p, bool f32, size_t e, float (&out)[Elt<DT>::kVec])
{
    constexpr int V = Elt<DT>::kVec;
    if (f32 || DT == NHP_F32) {
        const float* src = static_cast<const float*>(p) + e;
#pragma unroll
        for (int j = 0; j < V; j += 4) {
            const u32x4 r = load16(src + j);
#pragma unroll
            for (int i = 0; i < 4; ++i) out[j + i] = bitcast<float>(r[i]);
        }
    } else {
        chunk_to_float<DT>(load16(static_cast<const typename Elt<DT>::storage*>(p) + e), out);
    }
}

// The factor a row is multiplied by, from the sum of squares over its n statistic columns:
// 1 / (rms + eps) (eps_mode 1, the Python RMSNorm class), rsqrt(mean(x^2) + eps) (eps_mode 0) or
// 1 / max(||x||, eps) (eps_mode 2, ScaleNorm).
__device__ __forceinline__ float rms_inverse(float sumsq, float n, float eps, int eps_mode)
{
    if (eps_mode == 2) return 1.0f / fmaxf(sqrtf(sumsq), eps);
    if (eps_mode == 1) return 1.0f / (sqrtf(sumsq) * (1.0f / sqrtf(n)) + eps);
    return 1.0f / sqrtf(sumsq / n + eps);
}

// Factor of xhat * sum(g * xhat) in the RMSNorm backward (see norm_bwd_kernel).
__device__ __forceinline__ float rms_bwd_factor(float s2, float n, float inv, float eps, int eps_mode)
{
    if (eps_mode == 2) return inv < 1.0f / eps ? s2 : 0.0f;  // clamped norm: the factor does not depend on x
    float k2 = s2 / n;
    if (eps_mode == 1) {
        const float rho = 1.0f - eps * inv;
        k2 = rho > 0.0f ? k2 / rho : 0.0f;
    }
    return k2;
}

struct RowSlot {
    uint32_t row;
    int w;      // which of the row's W waves
    int group;  // row group inside the workgroup
    uint32_t l;
    bool ok;
};

// Which row (and which part of it) this thread works on in row block `rb`. A workgroup of G
// waves holds G / W row groups; with W = 1 a wave holds 64 / L rows of its own.
template <int W, int G>
__device__ __forceinline__ RowSlot locate(uint32_t rb, uint32_t rows, uint32_t L, uint32_t logL, int wave, int lane)
{
    static_assert(G % W == 0, "whole row groups");
    RowSlot s;
    s.l = (uint32_t)lane & (L - 1);
    if constexpr (W > 1) {
        s.group = wave / W;
        s.row = rb * (G / W) + (uint32_t)s.group;
        s.w = wave % W;
    } else {
        const uint32_t rows_per_wave = 64u >> logL;
        s.group = wave;
        s.row = (rb * G + (uint32_t)wave) * rows_per_wave + ((uint32_t)lane >> logL);
        s.w = 0;
    }
    s.ok = s.row < rows;
    return s;
}

// ---------------------------------------------------------------------------
// Forward
// ---------------------------------------------------------------------------
struct NormFwdArgs {
    void* y;
    float* mean;  // LayerNorm only, may be null
    float* rstd;  // LayerNorm: 1/sqrt(var + eps); RMSNorm: the factor x is multiplied by; may be null
    const void* x;
    const void* gamma;
    const void* beta;
    float eps;
    int eps_mode;
    uint32_t rows, cpr, L, logL;
    int params_f32;
    uint32_t stat;  // RMSNorm: the statistic is taken over the first `stat` columns
    // LayerNorm only, all null for a single norm: a second affine transform of the same normalised
    // row (two LayerNorms applied to one input share their statistics)
    void* y2;
    const void* gamma2;
    const void* beta2;
};

template <int DT, int K, int W, bool RMS>
__global__ void __launch_bounds__(((W > 1) ? W : kNormBlockWaves) * kWave)
norm_fwd_kernel(NormFwdArgs a)
{
    constexpr int V = Elt<DT>::kVec;
    using S = typename Elt<DT>::storage;
    constexpr int G = (W > 1) ? W : kNormBlockWaves;
    __shared__ float slots[2][16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const RowSlot rs = locate<W, G>(blockIdx.x, a.rows, a.L, a.logL, wave, lane);
    const size_t cols = (size_t)a.cpr * V;
    const float n = RMS ? (float)a.stat : (float)cols;
    const S* xr = static_cast<const S*>(a.x) + (size_t)rs.row * cols;
    S* yr = static_cast<S*>(a.y) + (size_t)rs.row * cols;

    u32x4 raw[K];
    bool live[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t cc = (uint32_t)(k * W + rs.w) * a.L + rs.l;
        live[k] = rs.ok && cc < a.cpr;
        raw[k] = u32x4{0, 0, 0, 0};
        if (live[k]) raw[k] = load16_stream(xr + (size_t)cc * V);
    }

    float mean = 0.0f, scale;
    if constexpr (!RMS) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float f[V];
            chunk_to_float<DT>(raw[k], f);
#pragma unroll
            for (int j = 0; j < V; ++j) s += f[j];
        }
        s = waves_sum<W>(lanes_sum(s, a.L), slots[0], rs.w, lane);
        mean = s / n;
    }
    {
        float q = 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (live[k]) {
                float f[V];
                chunk_to_float<DT>(raw[k], f);
                const uint32_t e0 = ((uint32_t)(k * W + rs.w) * a.L + rs.l) * V;
                if (!RMS || e0 + V <= a.stat) {
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        const float d = f[j] - mean;
                        q += d * d;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < V; ++j) q += (e0 + j < a.stat) ? f[j] * f[j] : 0.0f;
                }
            }
        }
        q = waves_sum<W>(lanes_sum(q, a.L), slots[1], rs.w, lane);
        scale = RMS ? rms_inverse(q, n, a.eps, a.eps_mode) : 1.0f / sqrtf(q / n + a.eps);
    }

#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (live[k]) {
            const uint32_t cc = (uint32_t)(k * W + rs.w) * a.L + rs.l;
            float f[V], g[V], b[V];
            chunk_to_float<DT>(raw[k], f);
#pragma unroll
            for (int j = 0; j < V; ++j) f[j] = (f[j] - mean) * scale;
            if (!RMS && a.y2 != nullptr) {
                float f2[V];
#pragma unroll
                for (int j = 0; j < V; ++j) f2[j] = f[j];
                if (a.gamma2 != nullptr) {
                    load_params<DT>(a.gamma2, a.params_f32 != 0, (size_t)cc * V, g);
#pragma unroll
                    for (int j = 0; j < V; ++j) f2[j] = f2[j] * g[j];
                }
                if (a.beta2 != nullptr) {
                    load_params<DT>(a.beta2, a.params_f32 != 0, (size_t)cc * V, b);
#pragma unroll
                    for (int j = 0; j < V; ++j) f2[j] = f2[j] + b[j];
                }
                store16_stream(static_cast<S*>(a.y2) + (size_t)rs.row * cols + (size_t)cc * V, float_to_chunk<DT>(f2));
            }
            if (a.gamma != nullptr) {
                load_params<DT>(a.gamma, a.params_f32 != 0, (size_t)cc * V, g);
#pragma unroll
                for (int j = 0; j < V; ++j) f[j] = RMS ? g[j] * f[j] : f[j] * g[j];
            }
            if (a.beta != nullptr) {
                load_params<DT>(a.beta, a.params_f32 != 0, (size_t)cc * V, b);
#pragma unroll
                for (int j = 0; j < V; ++j) f[j] = f[j] + b[j];
            }
            store16_stream(yr + (size_t)cc * V, float_to_chunk<DT>(f));
        }
    }
    if (rs.ok && rs.l == 0 && rs.w == 0) {
        if (!RMS && a.mean != nullptr) a.mean[rs.row] = mean;
        if (a.rstd != nullptr) a.rstd[rs.row] = scale;
    }
}

// One workgroup per row, elements strided over the threads, the row re-read for every pass.
__device__ __forceinline__ float block_sum_256(float v, float* slots)
{
    v = lanes_sum(v, 64);
    __syncthreads();  // slots may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    return (slots[0] + slots[1]) + (slots[2] + slots[3]);
}

template <int DT, bool RMS>
__global__ void __launch_bounds__(kNormScalarThreads)
norm_fwd_scalar_kernel(void* y, float* mean_out, float* rstd_out, const void* x, const void* gamma,
                       const void* beta, float eps, int eps_mode, uint64_t cols, uint64_t stat, int pdt,
                       void* y2, const void* gamma2, const void* beta2)
{
    __shared__ float slots[4];
    const uint64_t row = blockIdx.x;
    const int64_t base = (int64_t)(row * cols);
    const float n = RMS ? (float)stat : (float)cols;
    float mean = 0.0f;
    if (!RMS) {
        float s = 0.0f;
        for (uint64_t c = threadIdx.x; c < cols; c += kNormScalarThreads) s += Elt<DT>::load(x, base + (int64_t)c);
        mean = block_sum_256(s, slots) / n;
    }
    float q = 0.0f;
    for (uint64_t c = threadIdx.x; c < (RMS ? stat : cols); c += kNormScalarThreads) {
        const float d = Elt<DT>::load(x, base + (int64_t)c) - mean;
        q += d * d;
    }
    q = block_sum_256(q, slots);
    const float scale = RMS ? rms_inverse(q, n, eps, eps_mode) : 1.0f / sqrtf(q / n + eps);
    auto param = [&](const void* p, uint64_t c) {
        return pdt == NHP_F32 ? static_cast<const float*>(p)[c] : Elt<DT>::load(p, (int64_t)c);
    };
    for (uint64_t c = threadIdx.x; c < cols; c += kNormScalarThreads) {
        float f = (Elt<DT>::load(x, base + (int64_t)c) - mean) * scale;
        if (!RMS && y2 != nullptr) {
            float f2 = f;
            if (gamma2 != nullptr) f2 = f2 * param(gamma2, c);
            if (beta2 != nullptr) f2 = f2 + param(beta2, c);
            Elt<DT>::store(y2, base + (int64_t)c, f2);
        }
        if (gamma != nullptr) f = RMS ? param(gamma, c) * f : f * param(gamma, c);
        if (beta != nullptr) f = f + param(beta, c);
        Elt<DT>::store(y, base + (int64_t)c, f);
    }
    if (threadIdx.x == 0) {
        if (!RMS && mean_out != nullptr) mean_out[row] = mean;
        if (rstd_out != nullptr) rstd_out[row] = scale;
    }
}

// ---------------------------------------------------------------------------
// Backward
//   xhat = (x - mean) * rstd (RMSNorm: x * inv), g = dy * gamma
//   LayerNorm: dx = rstd * (g - (sum(g) + xhat * sum(g * xhat)) / cols)
//   RMSNorm:   dx = inv * (g - [c < stat] * xhat * sum(g * xhat) / (stat * rho)), rho = 1 for eps_mode 0
//              and 1 - eps * inv for eps_mode 1 (rho <= 0: the second term is dropped); eps_mode 2:
//              dx = inv * (g - xhat * sum(g * xhat)) while the norm is above eps, inv * g below
//   dgamma[c] = sum over rows of dy * xhat, dbeta[c] = sum over rows of dy
// ---------------------------------------------------------------------------
struct NormBwdArgs {
    void* dx;
    float* part_g;  // [gridDim.x, cols] partial sums for dgamma, or null (no parameter gradients)
    float* part_b;  // same for dbeta
    const void* dy;
    const void* x;
    const float* mean;
    const float* rstd;
    const void* gamma;
    float eps;
    int eps_mode;
    uint32_t rows, cpr, L, logL, row_blocks;
    int params_f32;
    uint32_t stat;  // RMSNorm: number of leading columns the statistic was taken over
    // PAIR kernels (two LayerNorms of one input): the second incoming gradient, its gamma and partial sums
    const void* dy2;
    const void* gamma2;
    float* part_g2;
    float* part_b2;
};

// Waves per workgroup of the backward kernel: as many row groups as the LDS buffer of the final
// accumulator reduction (K * V floats per thread, at most 32 KiB) and 512 threads allow (workgroups
// of 1024 threads measured slower), or the W waves of one row if that is more.
// Without parameter gradients (PARAMS = false: nothing is carried from row to row, a workgroup is only the
// unit that shares a barrier) at most 4 waves: the row groups of a workgroup then wait for each other less,
// 39.2 -> 34.9 us at [16384, 2048], 75.2 -> 67.9 us at [16384, 4096]. With parameter gradients smaller
// workgroups mean more partial rows and lose (42.3 -> 51.5 us at 2048 columns).
template <int K, int W, int V, bool PARAMS = true>
constexpr int bwd_waves()
{
    int g = 8192 / (K * V) / kWave;  // threads by the LDS bound, in waves
    const int cap = PARAMS ? 8 : 4;
    if (g > cap) g = cap;
    g = g / W * W;                    // whole row groups
    return g < W ? W : g;
}

// Row blocks in flight per iteration of the backward loop: two, or one where the registers of a second
// would cost a resident workgroup (two incoming gradients; rows of 10 or more KiB-segments: 93 instead of
// 145 VGPRs at K = 2, W = 8, 146 -> 130 us at [16384, 6144]).
constexpr int bwd_rows_in_flight(int k, int w, bool pair) { return (pair || k * w >= 10) ? 1 : 2; }

// PAIR (LayerNorm only): g = dy * gamma + dy2 * gamma2, one dx for both norms, and the parameter
// gradients of the second norm beside those of the first.
// PARAMS = false: no parameter gradients are wanted; the column sums and everything around them are left out.
template <int DT, int K, int W, bool RMS, bool PAIR = false, bool PARAMS = true, int U = bwd_rows_in_flight(K, W, PAIR)>
__global__ void __launch_bounds__((bwd_waves<K, W, Elt<DT>::kVec, PARAMS>() * kWave))
norm_bwd_kernel(NormBwdArgs a)
{
    static_assert(!PAIR || !RMS, "pairs of LayerNorms only");
    constexpr int V = Elt<DT>::kVec;
    constexpr int G = bwd_waves<K, W, V, PARAMS>();
    constexpr int T = G * kWave;
    constexpr int GROUPS = G / W;
    using S = typename Elt<DT>::storage;
    // [parity of the loop iteration][sum][row group][wave]: one barrier per iteration is enough when
    // consecutive iterations use different slots
    __shared__ float slots[2][2 * U][GROUPS > 1 ? GROUPS : 1][16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t cols = (size_t)a.cpr * V;
    const float n = RMS ? (float)a.stat : (float)cols;
    const bool param_grads = PARAMS && a.part_g != nullptr;

    // this thread's chunk columns do not depend on the row block
    const RowSlot first = locate<W, G>(0, a.rows, a.L, a.logL, wave, lane);
    uint32_t cc[K];
    bool col_live[K];
    bool stat_full[K];  // every column of the chunk took part in the statistic
    constexpr int K2 = PAIR ? K : 1;  // extent of the arrays only a pair uses
    float gam[K][V], gam2[K2][V];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        cc[k] = (uint32_t)(k * W + first.w) * a.L + first.l;
        col_live[k] = cc[k] < a.cpr;
        stat_full[k] = !RMS || (cc[k] + 1) * V <= a.stat;
#pragma unroll
        for (int j = 0; j < V; ++j) gam[k][j] = 1.0f;
        if (col_live[k] && a.gamma != nullptr) load_params<DT>(a.gamma, a.params_f32 != 0, (size_t)cc[k] * V, gam[k]);
        if constexpr (PAIR) {
#pragma unroll
            for (int j = 0; j < V; ++j) gam2[k][j] = 1.0f;
            if (col_live[k] && a.gamma2 != nullptr)
                load_params<DT>(a.gamma2, a.params_f32 != 0, (size_t)cc[k] * V, gam2[k]);
        }
    }

    float acc_g[K][V], acc_b[K][V], acc_g2[K2][V], acc_b2[K2][V];
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
        for (int j = 0; j < V; ++j) acc_g[k][j] = acc_b[k][j] = 0.0f;
#pragma unroll
    for (int k = 0; k < K2; ++k)
#pragma unroll
        for (int j = 0; j < V; ++j) acc_g2[k][j] = acc_b2[k][j] = 0.0f;

    // Every iteration takes U consecutive row blocks; all their loads are issued before the
    // first value is used (several rows in flight per thread without relying on a prefetch that
    // the compiler would have to track across the loop's back edge).
    int parity = 0;
    for (uint32_t rb0 = blockIdx.x * U; rb0 < a.row_blocks; rb0 += gridDim.x * U) {
        RowSlot rs[U];
        u32x4 rg[U][K], rx[U][K], rg2[U][K2];
        float mean[U], scale[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            rs[u] = locate<W, G>(rb0 + u, a.rows, a.L, a.logL, wave, lane);
            rs[u].ok = rs[u].ok && rb0 + u < a.row_blocks;
            const S* gr = static_cast<const S*>(a.dy) + (size_t)rs[u].row * cols;
            const S* xr = static_cast<const S*>(a.x) + (size_t)rs[u].row * cols;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                rg[u][k] = u32x4{0, 0, 0, 0};
                rx[u][k] = u32x4{0, 0, 0, 0};
                if constexpr (PAIR) rg2[u][k] = u32x4{0, 0, 0, 0};
                if (rs[u].ok && col_live[k]) {
                    rg[u][k] = load16_stream(gr + (size_t)cc[k] * V);
                    rx[u][k] = load16_stream(xr + (size_t)cc[k] * V);
                    if constexpr (PAIR)
                        rg2[u][k] = load16_stream(static_cast<const S*>(a.dy2) + (size_t)rs[u].row * cols + (size_t)cc[k] * V);
                }
            }
            mean[u] = 0.0f;
            scale[u] = 0.0f;
            if (rs[u].ok) {
                if (!RMS) mean[u] = a.mean[rs[u].row];
                scale[u] = a.rstd[rs[u].row];
            }
        }

        float s1[U], s2[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            s1[u] = s2[u] = 0.0f;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if (rs[u].ok && col_live[k]) {
                    float fg[V], fx[V], fg2[V];
                    chunk_to_float<DT>(rg[u][k], fg);
                    chunk_to_float<DT>(rx[u][k], fx);
                    if constexpr (PAIR) chunk_to_float<DT>(rg2[u][k], fg2);
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        const float xh = (fx[j] - mean[u]) * scale[u];
                        float g = fg[j] * gam[k][j];
                        if constexpr (PAIR) {
                            g = g + fg2[j] * gam2[k][j];
                            if constexpr (PARAMS) {
                                acc_g2[k][j] += fg2[j] * xh;
                                acc_b2[k][j] += fg2[j];
                            }
                        }
                        s1[u] += g;
                        s2[u] += g * xh;
                        if constexpr (PARAMS) {
                            acc_g[k][j] += fg[j] * xh;
                            acc_b[k][j] += fg[j];
                        }
                    }
                }
            }
            s1[u] = lanes_sum(s1[u], a.L);
            s2[u] = lanes_sum(s2[u], a.L);
        }
        if constexpr (W > 1) {
            // all sums of the iteration cross the rows' waves behind one barrier
            float(*mine)[GROUPS > 1 ? GROUPS : 1][16] = slots[parity];
            const int grp = rs[0].group, w = rs[0].w;
            if (lane == 0) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    mine[2 * u][grp][w] = s1[u];
                    mine[2 * u + 1][grp][w] = s2[u];
                }
            }
            __syncthreads();
#pragma unroll
            for (int u = 0; u < U; ++u) {
                s1[u] = mine[2 * u][grp][0];
                s2[u] = mine[2 * u + 1][grp][0];
#pragma unroll
                for (int i = 1; i < W; ++i) {
                    s1[u] += mine[2 * u][grp][i];
                    s2[u] += mine[2 * u + 1][grp][i];
                }
            }
            parity ^= 1;
        }

#pragma unroll
        for (int u = 0; u < U; ++u) {
            // LayerNorm: t = (s1 + xhat * s2) / n as c1 + xhat * c2 (no division per element)
            const float c1 = s1[u] / n;
            const float k2 = RMS ? rms_bwd_factor(s2[u], n, scale[u], a.eps, a.eps_mode) : s2[u] / n;
            S* dr = static_cast<S*>(a.dx) + (size_t)rs[u].row * cols;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if (rs[u].ok && col_live[k]) {
                    float fg[V], fx[V], o[V], fg2[V];
                    chunk_to_float<DT>(rg[u][k], fg);
                    chunk_to_float<DT>(rx[u][k], fx);
                    if constexpr (PAIR) chunk_to_float<DT>(rg2[u][k], fg2);
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        const float xh = (fx[j] - mean[u]) * scale[u];
                        float g = fg[j] * gam[k][j];
                        if constexpr (PAIR) g = g + fg2[j] * gam2[k][j];
                        float t = RMS ? xh * k2 : c1 + xh * k2;
                        if (RMS && !stat_full[k]) t = (cc[k] * V + j < a.stat) ? t : 0.0f;
                        o[j] = scale[u] * (g - t);
                    }
                    store16_stream(dr + (size_t)cc[k] * V, float_to_chunk<DT>(o));
                }
            }
        }
    }

    if (!param_grads) return;
    if constexpr (!PARAMS) {
        return;
    } else if constexpr (W > 1 && GROUPS == 1) {
        // one row group: every thread owns its columns alone
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (col_live[k]) {
                float* pg = a.part_g + (size_t)blockIdx.x * cols + (size_t)cc[k] * V;
                float* pb = a.part_b + (size_t)blockIdx.x * cols + (size_t)cc[k] * V;
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    pg[j] = acc_g[k][j];
                    pb[j] = acc_b[k][j];
                }
                if constexpr (PAIR) {
                    float* pg2 = a.part_g2 + (size_t)blockIdx.x * cols + (size_t)cc[k] * V;
                    float* pb2 = a.part_b2 + (size_t)blockIdx.x * cols + (size_t)cc[k] * V;
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        pg2[j] = acc_g2[k][j];
                        pb2[j] = acc_b2[k][j];
                    }
                }
            }
        }
    } else {
        // the threads that hold the same columns for other rows are `stride` apart; the first of
        // them adds the others up, in a fixed order
        const uint32_t stride = (W > 1) ? (uint32_t)(W * kWave) : a.L;
        __shared__ float red[K * V * T];
        for (int pass = 0; pass < (PAIR ? 4 : 2); ++pass) {
            __syncthreads();
#pragma unroll
            for (int k = 0; k < K; ++k)
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    float v = pass == 0 ? acc_g[k][j] : acc_b[k][j];
                    if constexpr (PAIR) {
                        if (pass == 2) v = acc_g2[k][j];
                        if (pass == 3) v = acc_b2[k][j];
                    }
                    red[(k * V + j) * T + threadIdx.x] = v;
                }
            __syncthreads();
            if (threadIdx.x < stride) {
                float* part = pass == 0 ? a.part_g : pass == 1 ? a.part_b : pass == 2 ? a.part_g2 : a.part_b2;
                float* dst = part + (size_t)blockIdx.x * cols;
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    if (col_live[k]) {
                        float o[V];
#pragma unroll
                        for (int j = 0; j < V; ++j) {
                            float s = red[(k * V + j) * T + threadIdx.x];
                            for (uint32_t t = threadIdx.x + stride; t < (uint32_t)T; t += stride)
                                s += red[(k * V + j) * T + t];
                            o[j] = s;
                        }
#pragma unroll
                        for (int j = 0; j < V; j += 4)
                            *reinterpret_cast<f32x4*>(dst + (size_t)cc[k] * V + j) = f32x4{o[j], o[j + 1], o[j + 2], o[j + 3]};
                    }
                }
            }
        }
    }
}

template <int DT, bool RMS>
__global__ void __launch_bounds__(kNormScalarThreads)
norm_bwd_scalar_kernel(void* dx, const void* dy, const void* x, const float* mean_in, const float* rstd_in,
                       const void* gamma, float eps, int eps_mode, uint64_t cols, uint64_t stat, int pdt,
                       const void* dy2, const void* gamma2)
{
    __shared__ float slots[4];
    const uint64_t row = blockIdx.x;
    const int64_t base = (int64_t)(row * cols);
    const float n = RMS ? (float)stat : (float)cols;
    const float mean = RMS ? 0.0f : mean_in[row];
    const float scale = rstd_in[row];
    auto pval = [&](const void* p, uint64_t c) {
        if (p == nullptr) return 1.0f;
        return pdt == NHP_F32 ? static_cast<const float*>(p)[c] : Elt<DT>::load(p, (int64_t)c);
    };
    // the incoming gradient times gamma; with a second LayerNorm of the same input the sum of both
    auto gval = [&](uint64_t c) {
        float g = Elt<DT>::load(dy, base + (int64_t)c) * pval(gamma, c);
        if (!RMS && dy2 != nullptr) g = g + Elt<DT>::load(dy2, base + (int64_t)c) * pval(gamma2, c);
        return g;
    };
    float s1 = 0.0f, s2 = 0.0f;
    for (uint64_t c = threadIdx.x; c < cols; c += kNormScalarThreads) {
        const float xh = (Elt<DT>::load(x, base + (int64_t)c) - mean) * scale;
        const float g = gval(c);
        s1 += g;
        s2 += g * xh;
    }
    s1 = block_sum_256(s1, slots);
    s2 = block_sum_256(s2, slots);
    const float k2 = RMS ? rms_bwd_factor(s2, n, scale, eps, eps_mode) : 0.0f;
    for (uint64_t c = threadIdx.x; c < cols; c += kNormScalarThreads) {
        const float xh = (Elt<DT>::load(x, base + (int64_t)c) - mean) * scale;
        const float g = gval(c);
        const float t = RMS ? (c < stat ? xh * k2 : 0.0f) : (s1 + xh * s2) / n;
        Elt<DT>::store(dx, base + (int64_t)c, scale * (g - t));
    }
}

// parameter gradients for the scalar path: one thread per column, rows in order
template <int DT, bool RMS>
__global__ void __launch_bounds__(kNormScalarThreads)
norm_param_grad_scalar_kernel(void* dgamma, void* dbeta, const void* dy, const void* x, const float* mean_in,
                              const float* rstd_in, uint64_t rows, uint64_t cols, int pdt)
{
    const uint64_t c = (uint64_t)blockIdx.x * kNormScalarThreads + threadIdx.x;
    if (c >= cols) return;
    float sg = 0.0f, sb = 0.0f;
    for (uint64_t r = 0; r < rows; ++r) {
        const float m = RMS ? 0.0f : mean_in[r];
        const float g = Elt<DT>::load(dy, (int64_t)(r * cols + c));
        sg += g * ((Elt<DT>::load(x, (int64_t)(r * cols + c)) - m) * rstd_in[r]);
        sb += g;
    }
    auto put = [&](void* p, float v) {
        if (p == nullptr) return;
        if (pdt == NHP_F32)
            static_cast<float*>(p)[c] = v;
        else
            Elt<DT>::store(p, (int64_t)c, v);
    };
    put(dgamma, sg);
    put(dbeta, sb);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct NormPlan {
    uint32_t L, logL;
    int K, W;
};

// (K, W) pairs that are compiled
#define NHP_NORM_GEOMETRIES(X) X(1, 1) X(2, 1) X(4, 1) X(1, 2) X(2, 2) X(1, 4) X(2, 4) X(2, 5) X(2, 8) X(4, 8) X(4, 16)
// forward only: rows of 5-6 and 12 chunks per lane (hidden sizes 2560, 3072, 6144) without idle waves
#define NHP_NORM_FWD_GEOMETRIES(X) X(2, 3) X(2, 6)

// Geometry for rows of cpr chunks: a wave reads 1-2 KiB of a row (1 KiB of each of its two
// inputs in the backward); returns false when the row does not fit.
static bool plan_norm(int64_t cpr, bool backward, NormPlan& p, bool pair = false)
{
    if (cpr < 1) return false;
    p.L = 1;
    p.logL = 0;
    while (p.L < 64 && (int64_t)p.L < cpr) {
        p.L *= 2;
        ++p.logL;
    }
    const int64_t segs = (cpr + p.L - 1) / p.L;  // 16-byte chunks per lane over the whole row
    // workgroups of 3, 5 and 6 waves measured 6-9 % faster than the next power of two at 2560, 3072 and 5120
    // columns in the forward; in the backward only the 5 waves at 5120 columns gain (8 %)
    static const int fwd_table[][2] = {{1, 1}, {2, 1}, {2, 2}, {2, 3}, {2, 4}, {2, 5}, {2, 6}, {2, 8}, {4, 8}, {4, 16}};
    static const int bwd_table[][2] = {{1, 1}, {1, 2}, {1, 4}, {2, 4}, {2, 5}, {2, 8}, {4, 8}, {4, 16}};
    // two incoming gradients: the 5 waves at 5120 columns lose (254 against 222 us)
    static const int pair_bwd_table[][2] = {{1, 1}, {1, 2}, {1, 4}, {2, 4}, {2, 8}, {4, 8}, {4, 16}};
    // a forward that writes two results: a whole row of up to 4 chunks per lane in one wave measured faster
    static const int pair_fwd_table[][2] = {{1, 1}, {2, 1}, {4, 1}, {2, 4}, {2, 8}, {4, 8}, {4, 16}};
    p.K = p.W = 0;
    const int(*table)[2] = backward ? (pair ? pair_bwd_table : bwd_table) : pair ? pair_fwd_table : fwd_table;
    const size_t count = backward ? (pair ? sizeof(pair_bwd_table) / sizeof(pair_bwd_table[0])
                                          : sizeof(bwd_table) / sizeof(bwd_table[0]))
                         : pair   ? sizeof(pair_fwd_table) / sizeof(pair_fwd_table[0])
                                  : sizeof(fwd_table) / sizeof(fwd_table[0]);
    for (size_t i = 0; i < count; ++i) {
        if ((int64_t)table[i][0] * table[i][1] >= segs) {
            p.K = table[i][0];
            p.W = table[i][1];
            break;
        }
    }
    const int tk = NHP_TUNED_INT("NHP_NORM_K", 0), tw = NHP_TUNED_INT("NHP_NORM_W", 0);
    if (tk > 0 && tw > 0 && (int64_t)tk * tw >= segs) {
        p.K = tk;
        p.W = tw;
    }
    return p.K != 0;
}

// Row blocks when a workgroup has `waves` waves.
static uint32_t norm_row_blocks(int64_t rows, const NormPlan& p, int waves)
{
    const int64_t rows_per_block = p.W > 1 ? waves / p.W : (int64_t)waves * (64 / p.L);
    return (uint32_t)((rows + rows_per_block - 1) / rows_per_block);
}

static int bwd_waves_of(const NormPlan& p, int v, bool params = true)
{
    int g = 8192 / (p.K * v) / kWave;
    const int cap = params ? 8 : 4;
    if (g > cap) g = cap;
    g = g / p.W * p.W;
    return g < p.W ? p.W : g;
}

// With parameter gradients the backward grid is bounded (every workgroup writes a partial row
// that the second kernel has to read): 4096 waves in all, 16 per CU.
constexpr uint32_t kNormBwdWaves = 4096;
// Compute units of an MI355X. The grid bounds below are whole rounds of workgroups over this many CUs; on a
// part with another count they stay correct and only lose the "no ragged last round" property.
constexpr uint32_t kCUs = 256;

static uint32_t norm_bwd_grid(uint32_t row_blocks, bool param_grads, int waves_per_block, int in_flight,
                              bool one_per_cu = false)
{
    row_blocks = (row_blocks + in_flight - 1) / in_flight;  // a workgroup takes that many row blocks per iteration
    if (!param_grads) return row_blocks;
    // a whole number of workgroups per CU: a ragged last round costs more than the waves it adds
    uint32_t cap = kNormBwdWaves / (uint32_t)waves_per_block / kCUs * kCUs;
    // two gradients and two chunks per lane, or four chunks per lane: 158-163 VGPRs, one 8-wave workgroup per
    // CU is resident; a second round of workgroups costs more than it brings (244 -> 225 us at [16384, 6144])
    if (cap == 0 || one_per_cu) cap = kCUs;
    cap = (uint32_t)NHP_TUNED_INT("NHP_NORM_GRID", (int)cap);
    return row_blocks < cap ? row_blocks : cap;
}

static bool param_dtype_ok(int dtype, int pdt) { return pdt == dtype || pdt == NHP_F32; }

// The second LayerNorm of a pair applied to one input (all null for a single norm).
struct NormSecond {
    void* y2 = nullptr;            // forward
    const void* gamma2 = nullptr;  // forward and backward
    const void* beta2 = nullptr;   // forward
    const void* dy2 = nullptr;     // backward
    void* dgamma2 = nullptr;       // backward
    void* dbeta2 = nullptr;        // backward
};

template <int DT, bool RMS>
static int norm_fwd(void* y, float* mean, float* rstd, const void* x, const void* gamma, const void* beta, float eps,
                    int eps_mode, int64_t rows, int64_t cols, int64_t stat, int pdt, hipStream_t st,
                    const NormSecond& second = NormSecond{})
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    NormPlan p;
    const bool params_aligned = ptr_aligned16(gamma) && ptr_aligned16(beta) && ptr_aligned16(second.gamma2) &&
                                ptr_aligned16(second.beta2) && ptr_aligned16(second.y2);
    if (cols % V == 0 && ptr_aligned16(x) && ptr_aligned16(y) && params_aligned && plan_norm(cols / V, false, p, second.y2 != nullptr)) {
        NormFwdArgs a{y, mean, rstd, x, gamma, beta, eps, eps_mode, (uint32_t)rows, (uint32_t)(cols / V),
                      p.L, p.logL, pdt == NHP_F32 ? 1 : 0, (uint32_t)stat, second.y2, second.gamma2, second.beta2};
        const int waves = p.W > 1 ? p.W : kNormBlockWaves;
        const uint32_t blocks = norm_row_blocks(rows, p, waves);
        const int threads = waves * kWave;
        if (!grid_fits(blocks, threads)) return NHP_ERR_SHAPE;
#define X(K_, W_)                                                                      \
    if (p.K == K_ && p.W == W_) {                                                      \
        norm_fwd_kernel<DT, K_, W_, RMS><<<blocks, threads, 0, st>>>(a);               \
        return launch_result();                                                        \
    }
        NHP_NORM_GEOMETRIES(X)
        NHP_NORM_FWD_GEOMETRIES(X)
#undef X
        return NHP_ERR_SHAPE;
    }
    if (!grid_fits(rows, kNormScalarThreads)) return NHP_ERR_SHAPE;
    norm_fwd_scalar_kernel<DT, RMS><<<(uint32_t)rows, kNormScalarThreads, 0, st>>>(
        y, mean, rstd, x, gamma, beta, eps, eps_mode, (uint64_t)cols, (uint64_t)stat, pdt, second.y2, second.gamma2,
        second.beta2);
    return launch_result();
}

static int64_t norm_workspace_bytes(int64_t rows, int64_t cols, int dtype, bool pair = false)
{
    const int v = dtype == NHP_F32 ? 4 : 8;
    NormPlan p;
    if (rows <= 0 || cols <= 0 || cols % v != 0 || !plan_norm(cols / v, true, p, pair)) return 0;
    const int waves = bwd_waves_of(p, v);
    // sized for one row block in flight, the variant with the most workgroups
    return 2 * (int64_t)norm_bwd_grid(norm_row_blocks(rows, p, waves), true, waves, 1) * cols * (int64_t)sizeof(float);
}

template <int DT, bool RMS>
static int norm_bwd(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x, const float* mean,
                    const float* rstd, const void* gamma, void* workspace, float eps, int eps_mode, int64_t rows,
                    int64_t cols, int64_t stat, int pdt, hipStream_t st, const NormSecond& second = NormSecond{},
                    uint32_t max_partial_rows = 0)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    NormPlan p;
    const bool pair = !RMS && second.dy2 != nullptr;
    const bool want_params = dgamma != nullptr || dbeta != nullptr || second.dgamma2 != nullptr || second.dbeta2 != nullptr;
    if (cols % V == 0 && ptr_aligned16(dx) && ptr_aligned16(dy) && ptr_aligned16(x) && ptr_aligned16(gamma) &&
        ptr_aligned16(second.dy2) && ptr_aligned16(second.gamma2) && ptr_aligned16(workspace) &&
        plan_norm(cols / V, true, p, pair)) {
        const int waves = bwd_waves_of(p, V, want_params);
        const uint32_t row_blocks = norm_row_blocks(rows, p, waves);
        uint32_t grid = norm_bwd_grid(row_blocks, want_params, waves, bwd_rows_in_flight(p.K, p.W, pair),
                                      (pair && p.K >= 2) || p.K >= 4);
        // a caller with a fixed workspace: fewer workgroups, each striding over more row blocks
        if (want_params && max_partial_rows != 0 && grid > max_partial_rows) grid = max_partial_rows;
        const size_t part = (size_t)grid * cols;
        float* part_g = want_params ? static_cast<float*>(workspace) : nullptr;
        float* part_b = want_params ? part_g + part : nullptr;
        float* part_g2 = (want_params && pair) ? part_g + 2 * part : nullptr;
        float* part_b2 = (want_params && pair) ? part_g + 3 * part : nullptr;
        NormBwdArgs a{dx, part_g, part_b, dy, x, mean, rstd, gamma, eps, eps_mode, (uint32_t)rows,
                      (uint32_t)(cols / V), p.L, p.logL, row_blocks, pdt == NHP_F32 ? 1 : 0, (uint32_t)stat,
                      second.dy2, second.gamma2, part_g2, part_b2};
        const int threads = waves * kWave;
        if (!grid_fits(grid, threads)) return NHP_ERR_SHAPE;
        bool launched = false;
#define X(K_, W_)                                                                      \
    if (!launched && p.K == K_ && p.W == W_) {                                         \
        if constexpr (!RMS) {                                                          \
            if (pair && want_params)                                                   \
                norm_bwd_kernel<DT, K_, W_, false, true, true><<<grid, threads, 0, st>>>(a); \
            else if (pair)                                                             \
                norm_bwd_kernel<DT, K_, W_, false, true, false><<<grid, threads, 0, st>>>(a); \
            else if (want_params)                                                      \
                norm_bwd_kernel<DT, K_, W_, false, false, true><<<grid, threads, 0, st>>>(a); \
            else                                                                       \
                norm_bwd_kernel<DT, K_, W_, false, false, false><<<grid, threads, 0, st>>>(a); \
        } else {                                                                       \
            if (want_params)                                                           \
                norm_bwd_kernel<DT, K_, W_, RMS, false, true><<<grid, threads, 0, st>>>(a); \
            else                                                                       \
                norm_bwd_kernel<DT, K_, W_, RMS, false, false><<<grid, threads, 0, st>>>(a); \
        }                                                                              \
        launched = true;                                                               \
    }
        NHP_NORM_GEOMETRIES(X)
#undef X
        if (!launched) return NHP_ERR_SHAPE;
        int rc = launch_result();
        if (rc != NHP_OK || !want_params) return rc;
        const dim3 fgrid((uint32_t)((cols + kFinishCols - 1) / kFinishCols), 2);
        partial_rows_sum_kernel<DT><<<fgrid, kFinishCols * kFinishSlices, 0, st>>>(dgamma, dbeta, part_g, part_b, grid, (uint32_t)cols,
                                                            pdt == NHP_F32 ? 1 : 0);
        rc = launch_result();
        if (rc != NHP_OK || !pair) return rc;
        partial_rows_sum_kernel<DT><<<fgrid, kFinishCols * kFinishSlices, 0, st>>>(
            second.dgamma2, second.dbeta2, part_g2, part_b2, grid, (uint32_t)cols, pdt == NHP_F32 ? 1 : 0);
        return launch_result();
    }
    if (!grid_fits(rows, kNormScalarThreads)) return NHP_ERR_SHAPE;
    norm_bwd_scalar_kernel<DT, RMS><<<(uint32_t)rows, kNormScalarThreads, 0, st>>>(
        dx, dy, x, mean, rstd, gamma, eps, eps_mode, (uint64_t)cols, (uint64_t)stat, pdt, second.dy2, second.gamma2);
    int rc = launch_result();
    if (rc != NHP_OK || !want_params) return rc;
    const uint32_t pblocks = (uint32_t)((cols + kNormScalarThreads - 1) / kNormScalarThreads);
    if (dgamma != nullptr || dbeta != nullptr) {
        norm_param_grad_scalar_kernel<DT, RMS><<<pblocks, kNormScalarThreads, 0, st>>>(
            dgamma, dbeta, dy, x, mean, rstd, (uint64_t)rows, (uint64_t)cols, pdt);
        rc = launch_result();
        if (rc != NHP_OK) return rc;
    }
    if (pair && (second.dgamma2 != nullptr || second.dbeta2 != nullptr)) {
        norm_param_grad_scalar_kernel<DT, RMS><<<pblocks, kNormScalarThreads, 0, st>>>(
            second.dgamma2, second.dbeta2, second.dy2, x, mean, rstd, (uint64_t)rows, (uint64_t)cols, pdt);
        rc = launch_result();
    }
    return rc;
}

static int norm_check(int64_t rows, int64_t cols, int dtype, int pdt)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    if (!param_dtype_ok(dtype, pdt)) return NHP_ERR_DTYPE;
    if (rows < 0 || cols < 0 || rows >= ((int64_t)1 << 31)) return NHP_ERR_SHAPE;
    if (rows > 0 && cols > ((int64_t)1 << 62) / rows) return NHP_ERR_SHAPE;
    return NHP_OK;
}

template <bool RMS>
static int norm_fwd_dispatch(void* y, float* mean, float* rstd, const void* x, const void* gamma, const void* beta,
                             float eps, int eps_mode, int64_t rows, int64_t cols, int64_t stat, int dtype, int pdt,
                             void* stream, const NormSecond& second = NormSecond{})
{
    if (int rc = norm_check(rows, cols, dtype, pdt)) return rc;
    if (RMS && (eps_mode < 0 || eps_mode > 2)) return NHP_ERR_SHAPE;
    if (rows == 0 || cols == 0) return NHP_OK;
    if (RMS && (stat < 1 || stat > cols)) return NHP_ERR_SHAPE;
    if (!y || !x) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case NHP_F16:
        return norm_fwd<NHP_F16, RMS>(y, mean, rstd, x, gamma, beta, eps, eps_mode, rows, cols, stat, pdt, st, second);
    case NHP_BF16:
        return norm_fwd<NHP_BF16, RMS>(y, mean, rstd, x, gamma, beta, eps, eps_mode, rows, cols, stat, pdt, st, second);
    default:
        return norm_fwd<NHP_F32, RMS>(y, mean, rstd, x, gamma, beta, eps, eps_mode, rows, cols, stat, pdt, st, second);
    }
}

template <bool RMS>
static int norm_bwd_dispatch(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x, const float* mean,
                             const float* rstd, const void* gamma, void* workspace, float eps, int eps_mode,
                             int64_t rows, int64_t cols, int64_t stat, int dtype, int pdt, void* stream,
                             const NormSecond& second = NormSecond{}, uint32_t max_partial_rows = 0)
{
    if (int rc = norm_check(rows, cols, dtype, pdt)) return rc;
    if (RMS && (eps_mode < 0 || eps_mode > 2)) return NHP_ERR_SHAPE;
    if (rows == 0 || cols == 0) return NHP_OK;
    if (RMS && (stat < 1 || stat > cols)) return NHP_ERR_SHAPE;
    if (!dx || !dy || !x || !rstd || (!RMS && !mean)) return NHP_ERR_NULL;
    const bool want_params = dgamma != nullptr || dbeta != nullptr || second.dgamma2 != nullptr || second.dbeta2 != nullptr;
    if (want_params && workspace == nullptr && norm_workspace_bytes(rows, cols, dtype) > 0) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case NHP_F16:
        return norm_bwd<NHP_F16, RMS>(dx, dgamma, dbeta, dy, x, mean, rstd, gamma, workspace, eps, eps_mode, rows,
                                      cols, stat, pdt, st, second, max_partial_rows);
    case NHP_BF16:
        return norm_bwd<NHP_BF16, RMS>(dx, dgamma, dbeta, dy, x, mean, rstd, gamma, workspace, eps, eps_mode, rows,
                                       cols, stat, pdt, st, second, max_partial_rows);
    default:
        return norm_bwd<NHP_F32, RMS>(dx, dgamma, dbeta, dy, x, mean, rstd, gamma, workspace, eps, eps_mode, rows,
                                      cols, stat, pdt, st, second, max_partial_rows);
    }
}

// ---------------------------------------------------------------------------
// Fixed scratch memory for nhp_layernorm_bwd_noalloc: the partial rows of the parameter
// gradients live in a device array that is part of the loaded code object, so that entry
// point needs no workspace from the caller and no allocation. Every GPU the library runs
// on holds its own copy of the array at its own address; host code never uses the array's
// name as an address (it is only a handle for hipGetSymbolAddress), always the pointer
// looked up once per device.
// ---------------------------------------------------------------------------
constexpr size_t kNoallocScratchBytes = NHP_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoallocScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
static void* scratch_ptr[kMaxDevices];  // per device, filled on the first call with that device current

// Address of the current device's copy of `scratch`; nullptr on failure.
static void* noalloc_scratch()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        scratch_ptr[dev] = p;
    }
    return scratch_ptr[dev];
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int nhp_layernorm_fwd(void* y, float* mean, float* rstd, const void* x, const void* gamma, const void* beta,
                      float eps, int64_t rows, int64_t cols, int dtype, int param_dtype, void* stream)
{
    return norm_fwd_dispatch<false>(y, mean, rstd, x, gamma, beta, eps, 0, rows, cols, cols, dtype, param_dtype,
                                    stream);
}

int nhp_layernorm_bwd(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x, const float* mean,
                      const float* rstd, const void* gamma, void* workspace, int64_t rows, int64_t cols, int dtype,
                      int param_dtype, void* stream)
{
    return norm_bwd_dispatch<false>(dx, dgamma, dbeta, dy, x, mean, rstd, gamma, workspace, 0.0f, 0, rows, cols,
                                    cols, dtype, param_dtype, stream);
}

int nhp_layernorm_bwd_noalloc(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x, const float* mean,
                              const float* rstd, const void* gamma, int64_t rows, int64_t cols, int dtype,
                              int param_dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    void* ws = nullptr;
    uint32_t max_partial_rows = 0;
    if ((dgamma != nullptr || dbeta != nullptr) && rows > 0 && cols > 0) {
        // The fixed array holds two fp32 partial rows (dgamma, dbeta) per workgroup: where nhp_layernorm_bwd
        // would use more workgroups than fit, this entry point launches fewer (each strides over more row
        // blocks; the sums are then formed in another order, within rounding of nhp_layernorm_bwd's).
        // Rows too long for even 8 workgroups are refused.
        const int64_t fit = (int64_t)kNoallocScratchBytes / (2 * cols * (int64_t)sizeof(float));
        if (fit < 8) return NHP_ERR_SCRATCH;
        max_partial_rows = (uint32_t)(fit < (int64_t)kNormBwdWaves ? fit : (int64_t)kNormBwdWaves);
        ws = noalloc_scratch();
        if (ws == nullptr) return NHP_ERR_LAUNCH;
    }
    return norm_bwd_dispatch<false>(dx, dgamma, dbeta, dy, x, mean, rstd, gamma, ws, 0.0f, 0, rows, cols, cols, dtype,
                                    param_dtype, stream, NormSecond{}, max_partial_rows);
}

int nhp_layernorm_pair_fwd(void* y1, void* y2, float* mean, float* rstd, const void* x, const void* gamma1,
                           const void* beta1, const void* gamma2, const void* beta2, float eps, int64_t rows,
                           int64_t cols, int dtype, int param_dtype, void* stream)
{
    if (rows > 0 && cols > 0 && !y2) return NHP_ERR_NULL;
    if (y1 != nullptr && y1 == y2) return NHP_ERR_ALIAS;
    NormSecond second;
    second.y2 = y2;
    second.gamma2 = gamma2;
    second.beta2 = beta2;
    return norm_fwd_dispatch<false>(y1, mean, rstd, x, gamma1, beta1, eps, 0, rows, cols, cols, dtype, param_dtype,
                                    stream, second);
}

int nhp_layernorm_pair_bwd(void* dx, void* dgamma1, void* dbeta1, void* dgamma2, void* dbeta2, const void* dy1,
                           const void* dy2, const void* x, const float* mean, const float* rstd, const void* gamma1,
                           const void* gamma2, void* workspace, int64_t rows, int64_t cols, int dtype,
                           int param_dtype, void* stream)
{
    if (rows > 0 && cols > 0 && !dy2) return NHP_ERR_NULL;
    NormSecond second;
    second.dy2 = dy2;
    second.gamma2 = gamma2;
    second.dgamma2 = dgamma2;
    second.dbeta2 = dbeta2;
    return norm_bwd_dispatch<false>(dx, dgamma1, dbeta1, dy1, x, mean, rstd, gamma1, workspace, 0.0f, 0, rows, cols,
                                    cols, dtype, param_dtype, stream, second);
}

int64_t nhp_layernorm_pair_bwd_workspace_bytes(int64_t rows, int64_t cols, int dtype)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return 0;
    return 2 * norm_workspace_bytes(rows, cols, dtype, true);
}

int nhp_rmsnorm_fwd(void* y, float* inv, const void* x, const void* scale, const void* offset, float eps,
                    int eps_mode, int64_t rows, int64_t cols, int dtype, int param_dtype, void* stream)
{
    return norm_fwd_dispatch<true>(y, nullptr, inv, x, scale, offset, eps, eps_mode, rows, cols, cols, dtype,
                                   param_dtype, stream);
}

int nhp_rmsnorm_partial_fwd(void* y, float* inv, const void* x, const void* scale, const void* offset, float eps,
                            int eps_mode, int64_t rows, int64_t cols, int64_t stat_cols, int dtype, int param_dtype,
                            void* stream)
{
    return norm_fwd_dispatch<true>(y, nullptr, inv, x, scale, offset, eps, eps_mode, rows, cols, stat_cols, dtype,
                                   param_dtype, stream);
}

int nhp_rmsnorm_bwd(void* dx, void* dscale, void* doffset, const void* dy, const void* x, const float* inv,
                    const void* scale, void* workspace, float eps, int eps_mode, int64_t rows, int64_t cols,
                    int dtype, int param_dtype, void* stream)
{
    return norm_bwd_dispatch<true>(dx, dscale, doffset, dy, x, nullptr, inv, scale, workspace, eps, eps_mode, rows,
                                   cols, cols, dtype, param_dtype, stream);
}

int nhp_rmsnorm_partial_bwd(void* dx, void* dscale, void* doffset, const void* dy, const void* x, const float* inv,
                            const void* scale, void* workspace, float eps, int eps_mode, int64_t rows, int64_t cols,
                            int64_t stat_cols, int dtype, int param_dtype, void* stream)
{
    return norm_bwd_dispatch<true>(dx, dscale, doffset, dy, x, nullptr, inv, scale, workspace, eps, eps_mode, rows,
                                   cols, stat_cols, dtype, param_dtype, stream);
}

int64_t nhp_norm_bwd_workspace_bytes(int64_t rows, int64_t cols, int dtype)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return 0;
    return norm_workspace_bytes(rows, cols, dtype);
}

}  // extern "C"
