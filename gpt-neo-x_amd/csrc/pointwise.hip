// Element-wise kernels of the transformer layer for gfx950: bias + tanh-GeLU
// (forward, backward with the bias gradient) and bias + residual add.
//
// Tensors are [rows, cols] with a [cols] bias. A workgroup of 256 threads
// covers TW 16-byte chunk columns (TW a power of two, at most 64: a wave reads
// 1 KiB of a row) by 256/TW * U rows per step; thread (tr, tc) keeps the bias
// values of chunk column tc in registers. Workgroups that are consecutive in
// launch order are adjacent along a row, so the memory touched at any moment
// is a band of whole rows that moves down the tensor.
//
// Arithmetic: operands are widened to fp32, the expression is evaluated in
// fp32 and the result is rounded once to the storage type -- what the
// reference's TorchScript-fused kernels do. The tanh-GeLU is evaluated through
// 1 / (1 + e^(2u)) with the hardware exp2 and reciprocal (see gelu_gate).

#include "common.hpp"
#include "colsum.hpp"

#include <cstdlib>

namespace nhp {

constexpr int kPwThreads = 256;

// tanh-GeLU of the reference (megatron/model/activations.py:79-97) with x^2 shared and tanh
// eliminated. With u = 0.79788456 x (1 + 0.044715 x^2), e = exp(2u) and s = 1 / (1 + e):
//   tanh(u) = 1 - 2s, so  gelu(x) = 0.5 x (1 + tanh u) = x (1 - s)
//   and, with 1 - tanh^2 = 4 s (1 - s) and the reference's polynomial 0.79788456 + 0.1070322243 x^2,
//   gelu'(x) = 0.5 x (1 - tanh^2)(0.79788456 + 0.1070322243 x^2) + 0.5 (1 + tanh u)
//            = (1 - s) + (1 - s) x s (1.59576912 + 0.2140644486 x^2).
// Two transcendental instructions (exp2, rcp) and 7 / 11 other operations per element instead of
// 17 / 27 for the expressions written out in source order: the backward was bound by the vector
// ALU, not by memory. 1 - s carries the same absolute error (about 2^-24) as the `1 + tanh` of the
// source order; e = inf gives s = 0 and the limits gelu = x, gelu' = 1.
__device__ __forceinline__ float gelu_gate(float x, float x2)
{
    // exp2 argument 2 log2(e) u, the constants folded
    const float w = __builtin_fmaf(2.0f * kLog2e * 0.79788456f * 0.044715f, x2, 2.0f * kLog2e * 0.79788456f);
    const float e = exp2_raw(x * w);
    return __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float gelu_fwd(float x)
{
    const float s = gelu_gate(x, x * x);
    return x * (1.0f - s);
}

__device__ __forceinline__ float gelu_grad(float x)
{
    const float x2 = x * x;
    const float s = gelu_gate(x, x2);
    const float poly = __builtin_fmaf(2.0f * 0.1070322243f, x2, 2.0f * 0.79788456f);
    // (1 - s) x and s poly are formed first: each factor that reaches 0 does so before it can meet an
    // overflowed partner, so the result is finite wherever x^2 is (the domain of the reference's expression)
    const float q = 1.0f - s;
    return __builtin_fmaf(q * x, s * poly, q);
}

enum PointOp {
    kGeluFwd = 0,        // out = gelu(a + bias)
    kGeluBwd = 1,        // out = gelu'(b + bias) * a
    kBiasAddResidual = 2, // out = b + (a + bias), b optional
    kColumnSum = 3        // nothing stored: only the column sums of a (with COLSUM)
};

// One element. `a`, `b`: the two tensor operands (b unused by kGeluFwd), `bv`: bias.
template <int OP>
__device__ __forceinline__ float point_op(float a, float b, float bv, bool has_b)
{
    if constexpr (OP == kGeluFwd) {
        return gelu_fwd(bv + a);
    } else if constexpr (OP == kGeluBwd) {
        return gelu_grad(bv + b) * a;
    } else {
        const float v = a + bv;
        return has_b ? b + v : v;
    }
}

template <int OP>
constexpr bool kNeedsB = (OP != kGeluFwd && OP != kColumnSum);

// ---------------------------------------------------------------------------
// Tiled kernel. Thread (tr, tc) of a workgroup owns chunk column
// blockIdx.x * TW + tc; one step of the workgroup covers TR * U consecutive
// rows (all loads of a step are issued before the first result is computed).
// Steps are numbered down the tensor and workgroup row y takes the steps
// y, y + gridDim.y, ...: with gridDim.y = number of steps every workgroup does
// one step, with fewer the resident workgroups sweep the tensor together,
// front to back, which is the order HBM likes.
// COLSUM: also accumulate, per chunk column, the sum of the *stored* (rounded)
// results over the workgroup's steps and write it to partial[blockIdx.y][cols]
// (fp32); a second kernel adds these up.
// ---------------------------------------------------------------------------
template <int DT, int OP, int TW, int U, bool COLSUM>
__global__ void __launch_bounds__(kPwThreads)
pointwise_kernel(void* out, const void* a, const void* b, const void* bias, float* partial, uint32_t rows,
                 uint32_t cpr, uint32_t steps)
{
    constexpr int V = Elt<DT>::kVec;
    constexpr int TR = kPwThreads / TW;
    using S = typename Elt<DT>::storage;
    const uint32_t tc = threadIdx.x % TW;
    const uint32_t tr = threadIdx.x / TW;
    const uint32_t cc = blockIdx.x * TW + tc;  // chunk column
    const bool live = cc < cpr;
    const size_t row_elems = (size_t)cpr * V;
    const bool has_b = kNeedsB<OP> && b != nullptr;

    float bv[V];
#pragma unroll
    for (int j = 0; j < V; ++j) bv[j] = 0.0f;
    if (live && bias != nullptr) chunk_to_float<DT>(load16(static_cast<const S*>(bias) + (size_t)cc * V), bv);

    float sums[V];
#pragma unroll
    for (int j = 0; j < V; ++j) sums[j] = 0.0f;

    // loads of one step; rows beyond the tensor leave zeros
    auto fetch = [&](uint32_t step, u32x4 (&ra)[U], u32x4 (&rb)[U]) {
        const uint32_t r = step * (TR * U) + tr;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t row = r + u * TR;
            const size_t off = (size_t)row * row_elems + (size_t)cc * V;
            ra[u] = u32x4{0, 0, 0, 0};
            rb[u] = u32x4{0, 0, 0, 0};
            if (row < rows) {
                ra[u] = load16_stream(static_cast<const S*>(a) + off);
                if (has_b) rb[u] = load16_stream(static_cast<const S*>(b) + off);
            }
        }
    };

    if (live) {
        for (uint32_t step = blockIdx.y; step < steps; step += gridDim.y) {
            // all loads of the step are issued before the first value is used
            u32x4 ra[U], rb[U];
            fetch(step, ra, rb);
            const uint32_t r = step * (TR * U) + tr;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t row = r + u * TR;
                if (row < rows) {
                    float fa[V], fb[V], fo[V];
                    chunk_to_float<DT>(ra[u], fa);
                    if constexpr (OP == kColumnSum) {
#pragma unroll
                        for (int j = 0; j < V; ++j) sums[j] += fa[j];
                        continue;
                    }
                    chunk_to_float<DT>(rb[u], fb);
#pragma unroll
                    for (int j = 0; j < V; ++j) fo[j] = point_op<OP>(fa[j], fb[j], bv[j], has_b);
                    const u32x4 packed = float_to_chunk<DT>(fo);
                    store16_stream(static_cast<S*>(out) + (size_t)row * row_elems + (size_t)cc * V, packed);
                    if constexpr (COLSUM) {
                        float stored[V];
                        chunk_to_float<DT>(packed, stored);
#pragma unroll
                        for (int j = 0; j < V; ++j) sums[j] += stored[j];
                    }
                }
            }
        }
    }

    if constexpr (COLSUM) {
        // combine the TR row-lanes of a chunk column in a fixed order
        __shared__ float lds[TR > 1 ? kPwThreads * V : 1];
        if constexpr (TR > 1) {
#pragma unroll
            for (int j = 0; j < V; ++j) lds[(tr * V + j) * TW + tc] = sums[j];
            __syncthreads();
            if (tr == 0) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    float s = lds[j * TW + tc];
                    for (int t = 1; t < TR; ++t) s += lds[(t * V + j) * TW + tc];
                    sums[j] = s;
                }
            }
        }
        if (tr == 0 && live) {
            float* dst = partial + (size_t)blockIdx.y * row_elems + (size_t)cc * V;
#pragma unroll
            for (int j = 0; j < V; j += 4)
                *reinterpret_cast<f32x4*>(dst + j) = f32x4{sums[j], sums[j + 1], sums[j + 2], sums[j + 3]};
        }
    }
}

// ---------------------------------------------------------------------------
// Scalar kernels for shapes the chunked layout cannot take (cols not a
// multiple of the chunk, unaligned pointers).
// ---------------------------------------------------------------------------
template <int DT, int OP>
__global__ void __launch_bounds__(kPwThreads)
pointwise_scalar_kernel(void* out, const void* a, const void* b, const void* bias, uint64_t total, uint64_t cols)
{
    const uint64_t i = (uint64_t)blockIdx.x * kPwThreads + threadIdx.x;
    if (i >= total) return;
    const bool has_b = kNeedsB<OP> && b != nullptr;
    const float bv = bias != nullptr ? Elt<DT>::load(bias, (int64_t)(i % cols)) : 0.0f;
    const float fa = Elt<DT>::load(a, (int64_t)i);
    const float fb = has_b ? Elt<DT>::load(b, (int64_t)i) : 0.0f;
    Elt<DT>::store(out, (int64_t)i, point_op<OP>(fa, fb, bv, has_b));
}

// ---------------------------------------------------------------------------
// The three bias_dropout_add calls of the parallel-residual layer (dropout off) in one pass, each call
// evaluated in fp32 and rounded once like nhp_bias_add_residual:
//   t1 = round(x1 + bias1), t3 = round(t1 + (x2 + bias2)), out = round(residual + t3).
// One step per workgroup, the tile shape of pointwise_kernel.
// ---------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void round_chunk(float (&v)[Elt<DT>::kVec])
{
    if constexpr (DT != NHP_F32) {
        const u32x4 packed = float_to_chunk<DT>(v);
        chunk_to_float<DT>(packed, v);
    }
}

template <int DT, int TW, int U>
__global__ void __launch_bounds__(kPwThreads)
residual_pair_kernel(void* out, const void* x1, const void* bias1, const void* x2, const void* bias2,
                     const void* residual, uint32_t rows, uint32_t cpr, uint32_t steps)
{
    constexpr int V = Elt<DT>::kVec;
    constexpr int TR = kPwThreads / TW;
    using S = typename Elt<DT>::storage;
    const uint32_t tc = threadIdx.x % TW;
    const uint32_t tr = threadIdx.x / TW;
    const uint32_t cc = blockIdx.x * TW + tc;
    if (cc >= cpr) return;
    const size_t row_elems = (size_t)cpr * V;
    // one step per workgroup unless the tensor has more steps than the grid may have rows
    for (uint32_t step = blockIdx.y; step < steps; step += gridDim.y) {
    u32x4 r1[U], r2[U], rr[U];
    const uint32_t r = step * (TR * U) + tr;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = r + u * TR;
        const size_t off = (size_t)row * row_elems + (size_t)cc * V;
        r1[u] = r2[u] = rr[u] = u32x4{0, 0, 0, 0};
        if (row < rows) {
            r1[u] = load16_stream(static_cast<const S*>(x1) + off);
            r2[u] = load16_stream(static_cast<const S*>(x2) + off);
            rr[u] = load16_stream(static_cast<const S*>(residual) + off);
        }
    }
    float b1[V], b2[V];
#pragma unroll
    for (int j = 0; j < V; ++j) b1[j] = b2[j] = 0.0f;
    if (bias1 != nullptr) chunk_to_float<DT>(load16(static_cast<const S*>(bias1) + (size_t)cc * V), b1);
    if (bias2 != nullptr) chunk_to_float<DT>(load16(static_cast<const S*>(bias2) + (size_t)cc * V), b2);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = r + u * TR;
        if (row < rows) {
            float t1[V], t2[V], fr[V];
            chunk_to_float<DT>(r1[u], t1);
            chunk_to_float<DT>(r2[u], t2);
            chunk_to_float<DT>(rr[u], fr);
            if (bias1 != nullptr) {
#pragma unroll
                for (int j = 0; j < V; ++j) t1[j] = t1[j] + b1[j];
                round_chunk<DT>(t1);
            }
#pragma unroll
            for (int j = 0; j < V; ++j) t1[j] = t1[j] + (t2[j] + b2[j]);
            round_chunk<DT>(t1);
#pragma unroll
            for (int j = 0; j < V; ++j) t1[j] = fr[j] + t1[j];
            store16_stream(static_cast<S*>(out) + (size_t)row * row_elems + (size_t)cc * V, float_to_chunk<DT>(t1));
        }
    }
    }
}

template <int DT>
__global__ void __launch_bounds__(kPwThreads)
residual_pair_scalar_kernel(void* out, const void* x1, const void* bias1, const void* x2, const void* bias2,
                            const void* residual, uint64_t total, uint64_t cols)
{
    const uint64_t i = (uint64_t)blockIdx.x * kPwThreads + threadIdx.x;
    if (i >= total) return;
    auto rounded = [](float v) {
        typename Elt<DT>::storage tmp;
        Elt<DT>::store(&tmp, 0, v);
        return Elt<DT>::load(&tmp, 0);
    };
    float t1 = Elt<DT>::load(x1, (int64_t)i), t2 = Elt<DT>::load(x2, (int64_t)i);
    if (bias1 != nullptr) t1 = rounded(t1 + Elt<DT>::load(bias1, (int64_t)(i % cols)));
    if (bias2 != nullptr) t2 = t2 + Elt<DT>::load(bias2, (int64_t)(i % cols));
    Elt<DT>::store(out, (int64_t)i, Elt<DT>::load(residual, (int64_t)i) + rounded(t1 + t2));
}

// one thread per column, rows in order (used after the scalar kernel has stored dx)
template <int DT>
__global__ void __launch_bounds__(kPwThreads)
column_sum_scalar_kernel(void* out, const void* dx, uint64_t rows, uint64_t cols)
{
    const uint64_t c = (uint64_t)blockIdx.x * kPwThreads + threadIdx.x;
    if (c >= cols) return;
    float s = 0.0f;
    for (uint64_t r = 0; r < rows; ++r) s += Elt<DT>::load(dx, (int64_t)(r * cols + c));
    Elt<DT>::store(out, (int64_t)c, s);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct TilePlan {
    int tw;          // chunk columns per workgroup (power of two <= 64)
    uint32_t steps;  // row steps of TR * U rows
    uint32_t col_tiles, grid_y;
};

static int elem_size(int dt) { return dt == NHP_F32 ? 4 : 2; }

constexpr int kPwU = 2;       // rows in flight per thread, one step per workgroup
constexpr int kPwColsumU = 4; // ... when a workgroup loops over steps (column sums)
constexpr int kPwMaxTw = 64;  // a wave reads 1 KiB of a row
// Dynamic LDS asked for only to bound the resident workgroups per CU: with two
// input tensors six workgroups per CU stream better than eight (measured).
constexpr uint32_t kPwLdsTwoInputs = 24576;
// With column sums the grid is bounded, so that the partial rows stay a few per cent of the traffic.
constexpr uint32_t kPwColsumGridY = 512;

// Tile shape for a [rows, cols] tensor of cpr chunks per row.
static TilePlan plan_tiles(int64_t rows, int64_t cpr, bool colsum)
{
    TilePlan p;
    p.tw = 1;
    const int max_tw = NHP_TUNED_INT("NHP_PW_TW", kPwMaxTw);
    while (p.tw < max_tw && p.tw < cpr) p.tw *= 2;
    const int64_t step_rows = (int64_t)(kPwThreads / p.tw) * (colsum ? kPwColsumU : kPwU);
    p.steps = (uint32_t)((rows + step_rows - 1) / step_rows);
    p.col_tiles = (uint32_t)((cpr + p.tw - 1) / p.tw);
    uint32_t cap = colsum ? (uint32_t)NHP_TUNED_INT("NHP_PW_GY", kPwColsumGridY) : 65535u;
    if (cap == 0 || cap > 65535u) cap = 65535u;
    p.grid_y = p.steps < cap ? p.steps : cap;
    return p;
}

template <int DT, int OP, bool COLSUM>
static int launch_tiled(void* out, const void* a, const void* b, const void* bias, float* partial, int64_t rows,
                        int64_t cpr, const TilePlan& p, hipStream_t st)
{
    launch_prepare();
    const dim3 grid(p.col_tiles, p.grid_y);
    if (!grid_fits((int64_t)p.col_tiles * p.grid_y, kPwThreads)) return NHP_ERR_SHAPE;
    const uint32_t lds = (uint32_t)NHP_TUNED_INT("NHP_PW_LDS", (kNeedsB<OP> && b != nullptr) ? kPwLdsTwoInputs : 0);
#define CASE_U(TW_, U_)                                                                                  \
        pointwise_kernel<DT, OP, TW_, U_, COLSUM><<<grid, kPwThreads, lds, st>>>(                        \
            out, a, b, bias, partial, (uint32_t)rows, (uint32_t)cpr, p.steps);
#define CASE(TW_)                                                                                        \
    case TW_:                                                                                            \
        CASE_U(TW_, (COLSUM ? kPwColsumU : kPwU))                                                        \
        break;
    switch (p.tw) {
        CASE(1) CASE(2) CASE(4) CASE(8) CASE(16) CASE(32) CASE(64)
    default:
        return NHP_ERR_SHAPE;
    }
#undef CASE
#undef CASE_U
    return launch_result();
}

// Runs OP over [rows, cols]; with dbias != nullptr (kGeluBwd only) also the column sums of the result.
template <int DT, int OP>
static int run_pointwise(void* out, const void* a, const void* b, const void* bias, void* dbias, float* workspace,
                         int64_t rows, int64_t cols, hipStream_t st)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    const bool chunked = cols % V == 0 && ptr_aligned16(out) && ptr_aligned16(a) && ptr_aligned16(b) &&
                         ptr_aligned16(bias) && ptr_aligned16(workspace) && rows < ((int64_t)1 << 31) &&
                         cols / V < ((int64_t)1 << 31);
    if (chunked) {
        const int64_t cpr = cols / V;
        if (dbias == nullptr)
            return launch_tiled<DT, OP, false>(out, a, b, bias, nullptr, rows, cpr, plan_tiles(rows, cpr, false), st);
        if constexpr (OP == kGeluBwd || OP == kColumnSum) {
            const TilePlan p = plan_tiles(rows, cpr, true);
            int rc = launch_tiled<DT, OP, true>(out, a, b, bias, workspace, rows, cpr, p, st);
            if (rc != NHP_OK) return rc;
            const int64_t blocks = (cols + kFinishCols - 1) / kFinishCols;
            if (!grid_fits(blocks, kFinishCols * kFinishSlices)) return NHP_ERR_SHAPE;
            partial_rows_sum_kernel<DT><<<dim3((uint32_t)blocks, 1), kFinishCols * kFinishSlices, 0, st>>>(
                dbias, nullptr, workspace, nullptr, p.grid_y, (uint32_t)cols, DT == NHP_F32 ? 1 : 0);
            return launch_result();
        }
        return NHP_ERR_SHAPE;
    }
    if constexpr (OP == kColumnSum) {
        if (!grid_fits((cols + kPwThreads - 1) / kPwThreads, kPwThreads)) return NHP_ERR_SHAPE;
        column_sum_scalar_kernel<DT><<<(uint32_t)((cols + kPwThreads - 1) / kPwThreads), kPwThreads, 0, st>>>(
            dbias, a, (uint64_t)rows, (uint64_t)cols);
        return launch_result();
    }
    const int64_t total = rows * cols;
    const int64_t blocks = (total + kPwThreads - 1) / kPwThreads;
    if (!grid_fits(blocks, kPwThreads)) return NHP_ERR_SHAPE;
    pointwise_scalar_kernel<DT, OP><<<(uint32_t)blocks, kPwThreads, 0, st>>>(out, a, b, bias, (uint64_t)total,
                                                                             (uint64_t)cols);
    int rc = launch_result();
    if (rc != NHP_OK || dbias == nullptr) return rc;
    column_sum_scalar_kernel<DT><<<(uint32_t)((cols + kPwThreads - 1) / kPwThreads), kPwThreads, 0, st>>>(
        dbias, out, (uint64_t)rows, (uint64_t)cols);
    return launch_result();
}

template <int DT>
static int run_residual_pair(void* out, const void* x1, const void* bias1, const void* x2, const void* bias2,
                             const void* residual, int64_t rows, int64_t cols, hipStream_t st)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    const bool chunked = cols % V == 0 && ptr_aligned16(out) && ptr_aligned16(x1) && ptr_aligned16(x2) &&
                         ptr_aligned16(residual) && ptr_aligned16(bias1) && ptr_aligned16(bias2) &&
                         rows < ((int64_t)1 << 31) && cols / V < ((int64_t)1 << 31);
    if (chunked) {
        const int64_t cpr = cols / V;
        const TilePlan p = plan_tiles(rows, cpr, false);
        if (!grid_fits((int64_t)p.col_tiles * p.grid_y, kPwThreads)) return NHP_ERR_SHAPE;
        const dim3 grid(p.col_tiles, p.grid_y);
#define CASE(TW_)                                                                                   \
    case TW_:                                                                                       \
        residual_pair_kernel<DT, TW_, kPwU><<<grid, kPwThreads, kPwLdsTwoInputs, st>>>(             \
            out, x1, bias1, x2, bias2, residual, (uint32_t)rows, (uint32_t)cpr, p.steps);           \
        break;
        switch (p.tw) {
            CASE(1) CASE(2) CASE(4) CASE(8) CASE(16) CASE(32) CASE(64)
        default:
            return NHP_ERR_SHAPE;
        }
#undef CASE
        return launch_result();
    }
    const int64_t total = rows * cols;
    const int64_t blocks = (total + kPwThreads - 1) / kPwThreads;
    if (!grid_fits(blocks, kPwThreads)) return NHP_ERR_SHAPE;
    residual_pair_scalar_kernel<DT><<<(uint32_t)blocks, kPwThreads, 0, st>>>(out, x1, bias1, x2, bias2, residual,
                                                                            (uint64_t)total, (uint64_t)cols);
    return launch_result();
}

template <int OP>
static int dispatch_pointwise(void* out, const void* a, const void* b, const void* bias, void* dbias,
                              float* workspace, int64_t rows, int64_t cols, int dtype, hipStream_t st)
{
    switch (dtype) {
    case NHP_F16:
        return run_pointwise<NHP_F16, OP>(out, a, b, bias, dbias, workspace, rows, cols, st);
    case NHP_BF16:
        return run_pointwise<NHP_BF16, OP>(out, a, b, bias, dbias, workspace, rows, cols, st);
    case NHP_F32:
        return run_pointwise<NHP_F32, OP>(out, a, b, bias, dbias, workspace, rows, cols, st);
    default:
        return NHP_ERR_DTYPE;
    }
}

static int check_shape(int64_t rows, int64_t cols, int dtype)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    if (rows < 0 || cols < 0) return NHP_ERR_SHAPE;
    if (rows > 0 && cols > ((int64_t)1 << 62) / rows) return NHP_ERR_SHAPE;
    return NHP_OK;
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int nhp_bias_gelu_fwd(void* out, const void* y, const void* bias, int64_t rows, int64_t cols, int dtype,
                      void* stream)
{
    if (int rc = check_shape(rows, cols, dtype)) return rc;
    if (rows == 0 || cols == 0) return NHP_OK;
    if (!out || !y) return NHP_ERR_NULL;
    return dispatch_pointwise<kGeluFwd>(out, y, nullptr, bias, nullptr, nullptr, rows, cols, dtype,
                                        static_cast<hipStream_t>(stream));
}

int64_t nhp_bias_gelu_bwd_workspace_bytes(int64_t rows, int64_t cols, int dtype)
{
    if (check_shape(rows, cols, dtype) != NHP_OK || rows == 0 || cols == 0) return 0;
    const int v = 16 / elem_size(dtype);
    if (cols % v != 0) return 0;  // the scalar path sums the stored result directly
    const TilePlan p = plan_tiles(rows, cols / v, true);
    return (int64_t)p.grid_y * cols * (int64_t)sizeof(float);
}

int nhp_bias_gelu_bwd(void* dx, const void* g, const void* y, const void* bias, void* dbias, void* workspace,
                      int64_t rows, int64_t cols, int dtype, void* stream)
{
    if (int rc = check_shape(rows, cols, dtype)) return rc;
    if (rows == 0 || cols == 0) return NHP_OK;  // dbias of an empty tensor is left untouched
    if (!dx || !g || !y) return NHP_ERR_NULL;
    if (dbias != nullptr && workspace == nullptr && nhp_bias_gelu_bwd_workspace_bytes(rows, cols, dtype) > 0)
        return NHP_ERR_NULL;
    if (dbias != nullptr && (dbias == dx || dbias == workspace)) return NHP_ERR_ALIAS;
    return dispatch_pointwise<kGeluBwd>(dx, g, y, bias, dbias, static_cast<float*>(workspace), rows, cols, dtype,
                                        static_cast<hipStream_t>(stream));
}

int64_t nhp_column_sum_workspace_bytes(int64_t rows, int64_t cols, int dtype)
{
    return nhp_bias_gelu_bwd_workspace_bytes(rows, cols, dtype);
}

int nhp_column_sum(void* out, const void* x, void* workspace, int64_t rows, int64_t cols, int dtype, void* stream)
{
    if (int rc = check_shape(rows, cols, dtype)) return rc;
    if (rows == 0 || cols == 0) return NHP_OK;  // the sums of an empty tensor are left untouched
    if (!out || !x) return NHP_ERR_NULL;
    if (workspace == nullptr && nhp_column_sum_workspace_bytes(rows, cols, dtype) > 0) return NHP_ERR_NULL;
    if (out == x || out == workspace) return NHP_ERR_ALIAS;
    return dispatch_pointwise<kColumnSum>(nullptr, x, nullptr, nullptr, out, static_cast<float*>(workspace), rows,
                                          cols, dtype, static_cast<hipStream_t>(stream));
}

int nhp_bias_add_residual(void* out, const void* x, const void* bias, const void* residual, int64_t rows,
                          int64_t cols, int dtype, void* stream)
{
    if (int rc = check_shape(rows, cols, dtype)) return rc;
    if (rows == 0 || cols == 0) return NHP_OK;
    if (!out || !x) return NHP_ERR_NULL;
    return dispatch_pointwise<kBiasAddResidual>(out, x, residual, bias, nullptr, nullptr, rows, cols, dtype,
                                                static_cast<hipStream_t>(stream));
}

int nhp_bias_add_residual_pair(void* out, const void* x1, const void* bias1, const void* x2, const void* bias2,
                               const void* residual, int64_t rows, int64_t cols, int dtype, void* stream)
{
    if (int rc = check_shape(rows, cols, dtype)) return rc;
    if (rows == 0 || cols == 0) return NHP_OK;
    if (!out || !x1 || !x2 || !residual) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case NHP_F16:
        return run_residual_pair<NHP_F16>(out, x1, bias1, x2, bias2, residual, rows, cols, st);
    case NHP_BF16:
        return run_residual_pair<NHP_BF16>(out, x1, bias1, x2, bias2, residual, rows, cols, st);
    default:
        return run_residual_pair<NHP_F32>(out, x1, bias1, x2, bias2, residual, rows, cols, st);
    }
}

}  // extern "C"
