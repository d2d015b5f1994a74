// Scaled causal / padding-masked softmax, forward and backward, for gfx950.
//
// Data layout: every tensor is a dense array of rows of n 16-bit elements
// (fp16 or bf16). A row is cut into 16-byte chunks of 8 elements. Chunk c of a
// row is owned by
//     iteration k, wave w, lane l   with   c = (k*W + w)*L + l
// where L lanes (a power of two <= 64) of a wave share a row, W waves of a
// workgroup share a row (W > 1 only when L == 64) and each lane keeps K chunks
// in registers. One wave-wide load therefore reads L*16 contiguous bytes per
// row, and a row is read from HBM exactly once and written exactly once.
//
//   n <= 256        : L = n/8 rounded up to a power of two, K = 1, 64/L rows per wave
//   n <= 2048       : one wave per row, K = 1..4
//   n <= 65536      : W = 2..16 waves per row, partial max / sum exchanged
//                     through 2*W floats of LDS
//   otherwise, or if n % 8 != 0 or a pointer is not 16-byte aligned:
//                     a scalar three-pass kernel (one workgroup per row).
//
// Arithmetic (fp32): z = x*scale, m = max z, e = 2^((z-m)*log2(e) + 64),
// p = e * (1 / sum e). The constant 64 scales every e of a row by 2^64, which
// cancels in p, and keeps e out of the range where v_exp_f32 flushes to zero
// down to 2^-190, so probabilities in the bf16 subnormal range are still produced.
//
// Masks are applied by index: in the causal kernels columns k > q are never
// loaded and are written as zeros; in the padding-mask kernel a chunk whose 8
// mask bytes are all 1 is not loaded.

#include "common.hpp"

namespace nhp {

constexpr float kExpBias = 64.0f;
constexpr float kMaskFill = -10000.0f;  // scaled_masked_softmax.h:180-184 of the reference

template <int L, int K, int W, int BW>
struct Geo {
    static_assert(W == 1 || L == 64, "several waves per row only with full-wave rows");
    static constexpr int kRowsPerWave = kWave / L;
    static constexpr int kRowsPerBlock = (W > 1) ? 1 : BW * kRowsPerWave;
    static constexpr int kThreads = ((W > 1) ? W : BW) * kWave;
    static constexpr bool kUniformRow = (L == 64);  // every lane of a wave is on the same row
};

// Column of the first element of the chunk held in register slot k.
template <int L, int W>
__device__ __forceinline__ uint32_t chunk_col(int k, int w, int l)
{
    return (uint32_t)((k * W + w) * L + l) * 8u;
}

// Row softmax over the register tile z[K][8]; entries that must not take part
// hold -inf. On return z holds the probabilities (fp32).
// `nk`: only slots k < nk hold finite values (a wave-uniform count).
template <int L, int K, int W>
__device__ __forceinline__ void softmax_tile(float (&z)[K][8], int nk, float* lds, int wave, int lane)
{
    float m = kNegInf;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (k < nk) {
#pragma unroll
            for (int j = 0; j < 8; ++j) m = fmaxf(m, z[k][j]);
        }
    }
    m = group_reduce<OpMax, L>(m);
    m = block_combine<OpMax, W>(m, lds, wave, lane);

    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (k < nk) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float e = exp2_raw(fmaf(z[k][j] - m, kLog2e, kExpBias));
                z[k][j] = e;
                sum += e;
            }
        }
    }
    sum = group_reduce<OpSum, L>(sum);
    sum = block_combine<OpSum, W>(sum, lds + 16, wave, lane);

    const float inv = 1.0f / sum;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (k < nk) {
#pragma unroll
            for (int j = 0; j < 8; ++j) z[k][j] *= inv;
        }
    }
}

// Locate the row this lane works on. Rows are numbered over the whole tensor;
// `q` is the row's index inside its [n_q, n] matrix.
template <typename G>
__device__ __forceinline__ void locate_row(uint32_t block, uint32_t rows_per_matrix, int wave, int lane,
                                           int lanes_per_row, uint32_t& row, uint32_t& q)
{
    const uint32_t row0 = block * (uint32_t)G::kRowsPerBlock;
    const uint32_t q0 = row0 % rows_per_matrix;  // scalar: depends on the block id only
    uint32_t local;
    if constexpr (G::kRowsPerBlock == 1) {
        local = 0;
    } else if constexpr (G::kUniformRow) {
        local = (uint32_t)wave;
    } else {
        local = (uint32_t)(wave * G::kRowsPerWave + lane / lanes_per_row);
    }
    row = row0 + local;
    q = q0 + local;
    while (q >= rows_per_matrix) q -= rows_per_matrix;
}

// ---------------------------------------------------------------------------
// Causal forward
// ---------------------------------------------------------------------------
template <int DT, int L, int K, int W, int BW>
__global__ void __launch_bounds__((Geo<L, K, W, BW>::kThreads))
causal_fwd_kernel(uint16_t* y, const uint16_t* x, float scale, uint32_t total_rows, uint32_t n)
{
    using G = Geo<L, K, W, BW>;
    __shared__ float lds[32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & (L - 1);
    const int w = (W > 1) ? wave : 0;

    uint32_t row, q;
    locate_row<G>(blockIdx.x, n, wave, lane, L, row, q);
    const bool ok = row < total_rows;
    const uint32_t valid = ok ? q + 1 : 0;  // columns [0, valid) take part

    const uint16_t* xr = x + (size_t)row * n;
    uint16_t* yr = y + (size_t)row * n;

    // Number of register slots that hold at least one valid column. For
    // full-wave rows this is wave-uniform; for shared waves K == 1.
    int nk;
    if constexpr (G::kUniformRow) {
        const int first = w * 512;
        nk = ((int)valid > first) ? ((int)valid - first + W * 512 - 1) / (W * 512) : 0;
        if (nk > K) nk = K;
    } else {
        nk = K;
    }

    u32x4 raw[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        raw[k] = u32x4{0, 0, 0, 0};
        if (k < nk && col < valid) raw[k] = load16_stream(xr + col);
    }

    float z[K][8];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (k < nk) {
            const uint32_t col = chunk_col<L, W>(k, w, l);
            float f[8];
            unpack8<DT>(raw[k], f);
#pragma unroll
            for (int j = 0; j < 8; ++j) z[k][j] = f[j] * scale;
            // only the slot that straddles `valid` (or lies beyond it) needs masking
            bool edge;
            if constexpr (G::kUniformRow) {
                edge = (uint32_t)((k * W + w + 1) * 512) > valid;
            } else {
                edge = true;
            }
            if (edge) {
#pragma unroll
                for (int j = 0; j < 8; ++j) z[k][j] = (col + j < valid) ? z[k][j] : kNegInf;
            }
        }
    }

    softmax_tile<L, K, W>(z, nk, lds, wave, lane);

#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        if (ok && col < n) {
            if (k < nk && col < valid) {
                store16_stream(yr + col, pack8<DT>(z[k]));
            } else {
                store16_stream(yr + col, u32x4{0, 0, 0, 0});
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Padding-mask forward. A wave owns the rows (b, q) of its lanes and walks
// over `heads_per_wave` heads with them, so the mask bytes of a row are
// fetched and decoded once per head group.
// ---------------------------------------------------------------------------
template <int DT, int L, int K, int W, int BW>
__global__ void __launch_bounds__((Geo<L, K, W, BW>::kThreads))
masked_fwd_kernel(uint16_t* y, const uint16_t* x, const uint8_t* mask, float scale,
                  uint32_t bq_rows, uint32_t sq, uint32_t np, uint32_t n,
                  uint32_t heads_per_wave, uint32_t head_groups, int mask_per_batch)
{
    using G = Geo<L, K, W, BW>;
    __shared__ float lds[2][32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & (L - 1);
    const int w = (W > 1) ? wave : 0;

    // head group varies fastest so that the blocks sharing mask rows are
    // neighbours in logical order, i.e. run on the same XCD back to back.
    const uint32_t id = xcd_swizzle(blockIdx.x, gridDim.x);
    const uint32_t hg = id % head_groups;
    const uint32_t rb = id / head_groups;

    uint32_t local;
    if constexpr (G::kRowsPerBlock == 1) {
        local = 0;
    } else if constexpr (G::kUniformRow) {
        local = (uint32_t)wave;
    } else {
        local = (uint32_t)(wave * G::kRowsPerWave + lane / L);
    }
    const uint32_t bq = rb * (uint32_t)G::kRowsPerBlock + local;
    const bool ok = bq < bq_rows;
    const uint32_t bi = bq / sq;
    const uint32_t qi = bq - bi * sq;
    const uint8_t* mrow = mask + (size_t)(mask_per_batch ? bq : qi) * n;

    // decode the mask once
    bool inb[K];    // chunk lies inside the row
    bool dead[K];   // all eight columns masked: the scores are not needed
    uint32_t mb[K][2];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        inb[k] = ok && col < n;
        mb[k][0] = 0;
        mb[k][1] = 0;
        if (inb[k]) {
            const u32x2 v = load8(mrow + col);
            mb[k][0] = v[0];
            mb[k][1] = v[1];
        }
        dead[k] = (mb[k][0] == 0x01010101u) && (mb[k][1] == 0x01010101u);
    }

    const uint32_t h_begin = hg * heads_per_wave;
    const uint32_t h_end = (h_begin + heads_per_wave < np) ? h_begin + heads_per_wave : np;
    for (uint32_t h = h_begin; h < h_end; ++h) {
        const size_t base = ((size_t)(bi * np + h) * sq + qi) * n;
        const uint16_t* xr = x + base;
        uint16_t* yr = y + base;

        u32x4 raw[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t col = chunk_col<L, W>(k, w, l);
            raw[k] = u32x4{0, 0, 0, 0};
            if (inb[k] && !dead[k]) raw[k] = load16_stream(xr + col);
        }

        float z[K][8];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float f[8];
            unpack8<DT>(raw[k], f);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t byte = (mb[k][j >> 2] >> (8 * (j & 3))) & 0xffu;
                const float v = (byte == 1u) ? kMaskFill : f[j] * scale;
                z[k][j] = inb[k] ? v : kNegInf;
            }
        }

        softmax_tile<L, K, W>(z, K, lds[h & 1], wave, lane);

#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t col = chunk_col<L, W>(k, w, l);
            if (inb[k]) store16_stream(yr + col, pack8<DT>(z[k]));
        }
    }
}

// ---------------------------------------------------------------------------
// Backward (causal and unmasked). dx = scale * (dy*y - y * sum(dy*y)).
// dy and y stay packed in registers between the two passes.
// ---------------------------------------------------------------------------
template <int DT, int L, int K, int W, int BW, bool CAUSAL>
__global__ void __launch_bounds__((Geo<L, K, W, BW>::kThreads))
softmax_bwd_kernel(uint16_t* dx, const uint16_t* dy, const uint16_t* y, float scale,
                   uint32_t total_rows, uint32_t n, uint32_t rows_per_matrix)
{
    using G = Geo<L, K, W, BW>;
    __shared__ float lds[32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & (L - 1);
    const int w = (W > 1) ? wave : 0;

    uint32_t row, q;
    locate_row<G>(blockIdx.x, rows_per_matrix, wave, lane, L, row, q);
    const bool ok = row < total_rows;
    const uint32_t valid = ok ? (CAUSAL ? q + 1 : n) : 0;

    const size_t base = (size_t)row * n;

    int nk;
    if constexpr (G::kUniformRow) {
        const int first = w * 512;
        nk = ((int)valid > first) ? ((int)valid - first + W * 512 - 1) / (W * 512) : 0;
        if (nk > K) nk = K;
    } else {
        nk = K;
    }

    u32x4 rg[K], ry[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        rg[k] = u32x4{0, 0, 0, 0};
        ry[k] = u32x4{0, 0, 0, 0};
        if (k < nk && col < valid) {
            rg[k] = load16_stream(dy + base + col);
            ry[k] = load16_stream(y + base + col);
            if (CAUSAL && col + 8 > valid) {
                // zero the elements at and beyond `valid` (both operands)
                const uint32_t rem = valid - col;  // 1..7
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t keep = (rem >= 2u * i + 2u) ? 0xffffffffu
                                          : (rem == 2u * i + 1u) ? 0x0000ffffu : 0u;
                    rg[k][i] &= keep;
                    ry[k][i] &= keep;
                }
            }
        }
    }

    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (k < nk) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s = fmaf(Half2<DT>::lo(rg[k][i]), Half2<DT>::lo(ry[k][i]), s);
                s = fmaf(Half2<DT>::hi(rg[k][i]), Half2<DT>::hi(ry[k][i]), s);
            }
        }
    }
    s = group_reduce<OpSum, L>(s);
    s = block_combine<OpSum, W>(s, lds, wave, lane);

    // what the formula gives where dy = y = 0 (masked columns): +0 for finite s
    const float zv = scale * fmaf(-0.0f, s, 0.0f);
    const uint32_t zw = Half2<DT>::pack(zv, zv);

#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        if (ok && col < n) {
            u32x4 o;
            if (k < nk && col < valid) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g0 = Half2<DT>::lo(rg[k][i]), y0 = Half2<DT>::lo(ry[k][i]);
                    const float g1 = Half2<DT>::hi(rg[k][i]), y1 = Half2<DT>::hi(ry[k][i]);
                    const float o0 = scale * fmaf(-y0, s, g0 * y0);
                    const float o1 = scale * fmaf(-y1, s, g1 * y1);
                    o[i] = Half2<DT>::pack(o0, o1);
                }
            } else {
                o = u32x4{zw, zw, zw, zw};
            }
            store16_stream(dx + base + col, o);
        }
    }
}

// ---------------------------------------------------------------------------
// Scalar kernels for rows the chunked layout cannot take (n % 8 != 0,
// unaligned pointers, n > 65536). One workgroup of 256 threads per row,
// the row is re-read from global memory (L2) for every pass.
// ---------------------------------------------------------------------------
constexpr int kScalarThreads = 256;

template <typename Op>
__device__ __forceinline__ float block_reduce_256(float v, float* slots)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    v = group_reduce<Op, 64>(v);
    __syncthreads();  // slots may still be read from a previous reduction
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    return Op::apply(Op::apply(slots[0], slots[1]), Op::apply(slots[2], slots[3]));
}

// MODE 0: causal, MODE 1: padding mask
template <int DT, int MODE>
__global__ void __launch_bounds__(kScalarThreads)
scalar_fwd_kernel(uint16_t* y, const uint16_t* x, const uint8_t* mask, float scale,
                  uint64_t n, uint64_t sq, uint64_t np, int mask_per_batch)
{
    __shared__ float slots[4];
    const uint64_t row = blockIdx.x;
    const uint64_t q = row % sq;
    const uint16_t* xr = x + row * n;
    uint16_t* yr = y + row * n;
    const uint8_t* mrow = nullptr;
    uint64_t valid = n;
    if (MODE == 0) {
        valid = q + 1;
    } else {
        const uint64_t bi = row / (sq * np);
        mrow = mask + (mask_per_batch ? (bi * sq + q) : q) * n;
    }

    float m = kNegInf;
    for (uint64_t c = threadIdx.x; c < valid; c += kScalarThreads) {
        float z = Half2<DT>::from_bits(xr[c]) * scale;
        if (MODE == 1 && mrow[c] == 1) z = kMaskFill;
        m = fmaxf(m, z);
    }
    m = block_reduce_256<OpMax>(m, slots);

    float sum = 0.0f;
    for (uint64_t c = threadIdx.x; c < valid; c += kScalarThreads) {
        float z = Half2<DT>::from_bits(xr[c]) * scale;
        if (MODE == 1 && mrow[c] == 1) z = kMaskFill;
        sum += exp2_raw(fmaf(z - m, kLog2e, kExpBias));
    }
    sum = block_reduce_256<OpSum>(sum, slots);
    const float inv = 1.0f / sum;

    // all reads of x are done before the first write of y (y may alias x)
    for (uint64_t c0 = 0; c0 < n; c0 += kScalarThreads) {
        const uint64_t c = c0 + threadIdx.x;
        float p = 0.0f;
        if (c < valid) {
            float z = Half2<DT>::from_bits(xr[c]) * scale;
            if (MODE == 1 && mrow[c] == 1) z = kMaskFill;
            p = exp2_raw(fmaf(z - m, kLog2e, kExpBias)) * inv;
        }
        if (c < n) yr[c] = Half2<DT>::to_bits(p);
    }
}

template <int DT, bool CAUSAL>
__global__ void __launch_bounds__(kScalarThreads)
scalar_bwd_kernel(uint16_t* dx, const uint16_t* dy, const uint16_t* y, float scale,
                  uint64_t n, uint64_t rows_per_matrix)
{
    __shared__ float slots[4];
    const uint64_t row = blockIdx.x;
    const uint64_t valid = CAUSAL ? (row % rows_per_matrix) + 1 : n;
    const uint16_t* gr = dy + row * n;
    const uint16_t* yr = y + row * n;
    uint16_t* dr = dx + row * n;

    float s = 0.0f;
    for (uint64_t c = threadIdx.x; c < valid; c += kScalarThreads)
        s = fmaf(Half2<DT>::from_bits(gr[c]), Half2<DT>::from_bits(yr[c]), s);
    s = block_reduce_256<OpSum>(s, slots);

    for (uint64_t c = threadIdx.x; c < n; c += kScalarThreads) {
        float g = 0.0f, p = 0.0f;
        if (c < valid) {
            g = Half2<DT>::from_bits(gr[c]);
            p = Half2<DT>::from_bits(yr[c]);
        }
        dr[c] = Half2<DT>::to_bits(scale * fmaf(-p, s, g * p));
    }
}

// ---------------------------------------------------------------------------
// Host side: geometry selection and launch
// ---------------------------------------------------------------------------
struct RowPlan {
    int L, K, W;
};

constexpr int64_t kMaxResidentRow = 65536;
constexpr int kBlockWaves = 4;  // waves per workgroup when a wave owns whole rows

static bool plan_row(int64_t n, RowPlan& p)
{
    if (n < 8 || n % 8 != 0 || n > kMaxResidentRow) return false;
    const int64_t chunks = n / 8;
    if (chunks <= 32) {
        int L = 1;
        while (L < chunks) L *= 2;
        p = {L, 1, 1};
        return true;
    }
    if (chunks <= 256) {
        p = {64, (int)((chunks + 63) / 64), 1};
        return true;
    }
    for (int W = 2; W <= 16; W *= 2) {
        const int64_t k = (chunks + 64 * W - 1) / (64 * W);
        if (k <= 4) {
            p = {64, k < 3 ? 3 : (int)k, W};
            return true;
        }
    }
    const int64_t k = (chunks + 1023) / 1024;
    p = {64, k <= 6 ? 6 : 8, 16};
    return true;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Invoke F<L, K, W>() for the plan. The list is the set of instantiated geometries.
#define NHP_FOR_PLAN(PLAN, CALL)                                     \
    do {                                                             \
        const int key_ = (PLAN).L * 10000 + (PLAN).K * 100 + (PLAN).W; \
        switch (key_) {                                              \
            case 10101: CALL(1, 1, 1); break;                        \
            case 20101: CALL(2, 1, 1); break;                        \
            case 40101: CALL(4, 1, 1); break;                        \
            case 80101: CALL(8, 1, 1); break;                        \
            case 160101: CALL(16, 1, 1); break;                      \
            case 320101: CALL(32, 1, 1); break;                      \
            case 640101: CALL(64, 1, 1); break;                      \
            case 640201: CALL(64, 2, 1); break;                      \
            case 640301: CALL(64, 3, 1); break;                      \
            case 640401: CALL(64, 4, 1); break;                      \
            case 640302: CALL(64, 3, 2); break;                      \
            case 640402: CALL(64, 4, 2); break;                      \
            case 640304: CALL(64, 3, 4); break;                      \
            case 640404: CALL(64, 4, 4); break;                      \
            case 640308: CALL(64, 3, 8); break;                      \
            case 640408: CALL(64, 4, 8); break;                      \
            case 640316: CALL(64, 3, 16); break;                     \
            case 640416: CALL(64, 4, 16); break;                     \
            case 640616: CALL(64, 6, 16); break;                     \
            case 640816: CALL(64, 8, 16); break;                     \
            default: return NHP_ERR_SHAPE;                           \
        }                                                            \
    } while (0)

static inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? NHP_OK : NHP_ERR_LAUNCH;
}

constexpr int64_t kMaxRows = (int64_t)1 << 31;  // row and block ids are 32-bit on the device

template <int DT>
static int causal_fwd(void* y, const void* x, float scale, int64_t batches, int64_t n, hipStream_t st)
{
    const int64_t rows = batches * n;
    RowPlan p;
    uint16_t* yp = static_cast<uint16_t*>(y);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    if (plan_row(n, p) && aligned16(x) && aligned16(y)) {
#define CALL(L_, K_, W_)                                                                   \
    {                                                                                      \
        using G = Geo<L_, K_, W_, kBlockWaves>;                                            \
        const uint32_t blocks = (uint32_t)((rows + G::kRowsPerBlock - 1) / G::kRowsPerBlock); \
        causal_fwd_kernel<DT, L_, K_, W_, kBlockWaves><<<blocks, G::kThreads, 0, st>>>(    \
            yp, xp, scale, (uint32_t)rows, (uint32_t)n);                                   \
    }
        NHP_FOR_PLAN(p, CALL);
#undef CALL
    } else {
        scalar_fwd_kernel<DT, 0><<<(uint32_t)rows, kScalarThreads, 0, st>>>(
            yp, xp, nullptr, scale, (uint64_t)n, (uint64_t)n, 1, 0);
    }
    return launch_status();
}

template <int DT, bool CAUSAL>
static int softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows, int64_t n,
                       int64_t rows_per_matrix, hipStream_t st)
{
    RowPlan p;
    uint16_t* dxp = static_cast<uint16_t*>(dx);
    const uint16_t* dyp = static_cast<const uint16_t*>(dy);
    const uint16_t* yp = static_cast<const uint16_t*>(y);
    if (plan_row(n, p) && aligned16(dx) && aligned16(dy) && aligned16(y)) {
#define CALL(L_, K_, W_)                                                                   \
    {                                                                                      \
        using G = Geo<L_, K_, W_, kBlockWaves>;                                            \
        const uint32_t blocks = (uint32_t)((rows + G::kRowsPerBlock - 1) / G::kRowsPerBlock); \
        softmax_bwd_kernel<DT, L_, K_, W_, kBlockWaves, CAUSAL><<<blocks, G::kThreads, 0, st>>>( \
            dxp, dyp, yp, scale, (uint32_t)rows, (uint32_t)n, (uint32_t)rows_per_matrix);  \
    }
        NHP_FOR_PLAN(p, CALL);
#undef CALL
    } else {
        scalar_bwd_kernel<DT, CAUSAL><<<(uint32_t)rows, kScalarThreads, 0, st>>>(
            dxp, dyp, yp, scale, (uint64_t)n, (uint64_t)rows_per_matrix);
    }
    return launch_status();
}

// Heads a wave walks over with one decoded mask row: as many as possible
// while the grid still holds several waves per SIMD of the 256 CUs.
static uint32_t pick_heads_per_wave(int64_t bq_row_blocks, int64_t np, int waves_per_block)
{
    const int64_t want_waves = 256 * 4 * 8 * 4;  // four full rounds of 8 waves per SIMD
    int64_t hpw = np;
    while (hpw > 1 && bq_row_blocks * waves_per_block * ((np + hpw - 1) / hpw) < want_waves)
        hpw = (hpw + 1) / 2;
    return (uint32_t)hpw;
}

template <int DT>
static int masked_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b, int64_t np,
                      int64_t sq, int64_t n, int64_t pad_batches, hipStream_t st)
{
    const int64_t bq_rows = b * sq;
    const int per_batch = (pad_batches != 1) ? 1 : 0;
    RowPlan p;
    uint16_t* yp = static_cast<uint16_t*>(y);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const bool mask_ok = (reinterpret_cast<uintptr_t>(mask) & 7u) == 0;
    if (plan_row(n, p) && aligned16(x) && aligned16(y) && mask_ok) {
#define CALL(L_, K_, W_)                                                                   \
    {                                                                                      \
        using G = Geo<L_, K_, W_, kBlockWaves>;                                            \
        const int64_t rb = (bq_rows + G::kRowsPerBlock - 1) / G::kRowsPerBlock;            \
        const uint32_t hpw = pick_heads_per_wave(rb, np, G::kThreads / kWave);             \
        const uint32_t hgs = (uint32_t)((np + hpw - 1) / hpw);                             \
        if (rb * hgs >= kMaxRows) return NHP_ERR_SHAPE;                                    \
        masked_fwd_kernel<DT, L_, K_, W_, kBlockWaves><<<(uint32_t)(rb * hgs), G::kThreads, 0, st>>>( \
            yp, xp, mask, scale, (uint32_t)bq_rows, (uint32_t)sq, (uint32_t)np, (uint32_t)n, hpw, hgs, \
            per_batch);                                                                    \
    }
        NHP_FOR_PLAN(p, CALL);
#undef CALL
    } else {
        scalar_fwd_kernel<DT, 1><<<(uint32_t)(b * np * sq), kScalarThreads, 0, st>>>(
            yp, xp, mask, scale, (uint64_t)n, (uint64_t)sq, (uint64_t)np, per_batch);
    }
    return launch_status();
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int64_t nhp_softmax_max_resident_row(void) { return kMaxResidentRow; }

int nhp_causal_softmax_fwd(void* y, const void* x, float scale, int64_t attn_batches, int64_t seq_len,
                           int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    if (attn_batches < 0 || seq_len < 0) return NHP_ERR_SHAPE;
    if (attn_batches == 0 || seq_len == 0) return NHP_OK;
    if (attn_batches > kMaxRows / seq_len - 1) return NHP_ERR_SHAPE;
    if (!x || !y) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dtype == NHP_BF16 ? causal_fwd<NHP_BF16>(y, x, scale, attn_batches, seq_len, st)
                             : causal_fwd<NHP_F16>(y, x, scale, attn_batches, seq_len, st);
}

int nhp_causal_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                           int64_t seq_len, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    if (attn_batches < 0 || seq_len < 0) return NHP_ERR_SHAPE;
    if (attn_batches == 0 || seq_len == 0) return NHP_OK;
    if (attn_batches > kMaxRows / seq_len - 1) return NHP_ERR_SHAPE;
    if (!dx || !dy || !y) return NHP_ERR_NULL;
    if (dx == y) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t rows = attn_batches * seq_len;
    return dtype == NHP_BF16
               ? softmax_bwd<NHP_BF16, true>(dx, dy, y, scale, rows, seq_len, seq_len, st)
               : softmax_bwd<NHP_F16, true>(dx, dy, y, scale, rows, seq_len, seq_len, st);
}

int nhp_masked_softmax_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b,
                           int64_t np, int64_t sq, int64_t sk, int64_t pad_batches, int dtype,
                           void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    if (b < 0 || np < 0 || sq < 0 || sk < 0) return NHP_ERR_SHAPE;
    if (b == 0 || np == 0 || sq == 0 || sk == 0) return NHP_OK;
    if (pad_batches != 1 && pad_batches != b) return NHP_ERR_PAD_BATCHES;
    if (b > kMaxRows / np - 1 || b * np > kMaxRows / sq - 1) return NHP_ERR_SHAPE;
    if (!x || !y || !mask) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dtype == NHP_BF16 ? masked_fwd<NHP_BF16>(y, x, mask, scale, b, np, sq, sk, pad_batches, st)
                             : masked_fwd<NHP_F16>(y, x, mask, scale, b, np, sq, sk, pad_batches, st);
}

int nhp_masked_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows, int64_t sk,
                           int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    if (rows < 0 || sk < 0) return NHP_ERR_SHAPE;
    if (rows == 0 || sk == 0) return NHP_OK;
    if (rows >= kMaxRows) return NHP_ERR_SHAPE;
    if (!dx || !dy || !y) return NHP_ERR_NULL;
    if (dx == y) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // rows_per_matrix only matters for the causal variant; any non-zero value works here
    return dtype == NHP_BF16 ? softmax_bwd<NHP_BF16, false>(dx, dy, y, scale, rows, sk, rows, st)
                             : softmax_bwd<NHP_F16, false>(dx, dy, y, scale, rows, sk, rows, st);
}

int nhp_softmax_batch_per_block(int64_t query_seq_len, int64_t key_seq_len, int64_t batches,
                                int64_t attn_heads)
{
    (void)query_seq_len;
    (void)batches;
    (void)attn_heads;
    if (key_seq_len < 1) return NHP_ERR_SHAPE;
    int64_t pow2 = 1;
    while (pow2 < key_seq_len) pow2 *= 2;
    const int64_t warp = pow2 < kWave ? pow2 : kWave;
    const int64_t rows_per_warp = pow2 <= 128 ? 2 : 1;
    return (int)((128 / warp) * rows_per_warp);
}

}  // extern "C"
