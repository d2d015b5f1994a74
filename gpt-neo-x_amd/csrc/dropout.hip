// bias + dropout + residual add with dropout active, and the backward of the
// dropout, for gfx950.
//
//   forward:  out = residual + keep * (x + bias) / (1 - p)
//   backward: dx  = keep * g / (1 - p)
//
// The keep mask is never stored: element e (flat index in the [rows, cols]
// tensor) is kept when bits 16 * (e % 8) .. of the Philox4x32-10 output for
// counter (e / 8, offset) and key `seed` are below round((1 - p) * 65536), so
// forward and backward regenerate the same mask from (seed, offset). One
// Philox call serves one 16-byte chunk of 16-bit data.
//
// Launch shape: the one-step tiles of the other element-wise kernels.

#include "common.hpp"

#include <cstdlib>

namespace nhp {

constexpr int kDropThreads = 256;
constexpr int kDropU = 2;
constexpr int kDropMaxTw = 64;

struct DropArgs {
    void* out;
    const void* a;         // x (forward) or g (backward)
    const void* residual;  // forward only, may be null
    const void* bias;      // forward only, may be null
    uint32_t rows, cpr;
    uint32_t threshold;    // keep when random16 < threshold
    float scale;           // 1 / (1 - p)
    uint32_t seed_lo, seed_hi, off_lo, off_hi;
};

template <int DT, int TW>
__global__ void __launch_bounds__(kDropThreads)
dropout_kernel(DropArgs d)
{
    constexpr int V = Elt<DT>::kVec;
    constexpr int U = kDropU;
    constexpr int TR = kDropThreads / TW;
    using S = typename Elt<DT>::storage;
    const uint32_t tc = threadIdx.x % TW;
    const uint32_t tr = threadIdx.x / TW;
    const uint32_t cc = blockIdx.x * TW + tc;
    if (cc >= d.cpr) return;
    const size_t row_elems = (size_t)d.cpr * V;
    const size_t col = (size_t)cc * V;

    float bv[V];
#pragma unroll
    for (int j = 0; j < V; ++j) bv[j] = 0.0f;
    if (d.bias != nullptr) chunk_to_float<DT>(load16(static_cast<const S*>(d.bias) + col), bv);

    const uint32_t r0 = blockIdx.y * (TR * U) + tr;
    u32x4 ra[U], rr[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = r0 + u * TR;
        ra[u] = rr[u] = u32x4{0, 0, 0, 0};
        if (row < d.rows) {
            ra[u] = load16_stream(static_cast<const S*>(d.a) + (size_t)row * row_elems + col);
            if (d.residual != nullptr) rr[u] = load16_stream(static_cast<const S*>(d.residual) + (size_t)row * row_elems + col);
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = r0 + u * TR;
        if (row < d.rows) {
            const uint64_t e0 = (uint64_t)row * row_elems + col;  // flat index of the chunk's first element
            const uint64_t group = e0 >> 3;
            const Philox rnd = philox4x32_10((uint32_t)group, (uint32_t)(group >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi);
            const int base = (int)(e0 & 7u);  // 0, or 4 for the second fp32 chunk of a group
            float fa[V], fr[V], o[V];
            chunk_to_float<DT>(ra[u], fa);
            chunk_to_float<DT>(rr[u], fr);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const bool keep = random16(rnd, base + j) < d.threshold;
                const float v = keep ? (fa[j] + bv[j]) * d.scale : 0.0f;
                o[j] = d.residual != nullptr ? fr[j] + v : v;
            }
            store16_stream(static_cast<S*>(d.out) + (size_t)row * row_elems + col, float_to_chunk<DT>(o));
        }
    }
}

template <int DT>
__global__ void __launch_bounds__(kDropThreads)
dropout_scalar_kernel(DropArgs d, uint64_t total, uint64_t cols)
{
    const uint64_t e = (uint64_t)blockIdx.x * kDropThreads + threadIdx.x;
    if (e >= total) return;
    const uint64_t group = e >> 3;
    const Philox rnd = philox4x32_10((uint32_t)group, (uint32_t)(group >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi);
    const bool keep = random16(rnd, (int)(e & 7u)) < d.threshold;
    float v = Elt<DT>::load(d.a, (int64_t)e);
    if (d.bias != nullptr) v = v + Elt<DT>::load(d.bias, (int64_t)(e % cols));
    v = keep ? v * d.scale : 0.0f;
    if (d.residual != nullptr) v = Elt<DT>::load(d.residual, (int64_t)e) + v;
    Elt<DT>::store(d.out, (int64_t)e, v);
}

template <int DT>
static int dropout_launch(DropArgs d, int64_t rows, int64_t cols, hipStream_t st)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    const bool chunked = cols % V == 0 && ptr_aligned16(d.out) && ptr_aligned16(d.a) && ptr_aligned16(d.residual) &&
                         ptr_aligned16(d.bias) && rows < ((int64_t)1 << 31) && cols / V < ((int64_t)1 << 31);
    if (chunked) {
        const int64_t cpr = cols / V;
        int tw = 1;
        while (tw < kDropMaxTw && tw < cpr) tw *= 2;
        const int64_t step_rows = (int64_t)(kDropThreads / tw) * kDropU;
        const int64_t steps = (rows + step_rows - 1) / step_rows;
        const int64_t col_tiles = (cpr + tw - 1) / tw;
        if (steps <= 65535) {  // grid.y limit; taller tensors take the scalar kernel
            if (!grid_fits(col_tiles * steps, kDropThreads)) return NHP_ERR_SHAPE;
            d.rows = (uint32_t)rows;
            d.cpr = (uint32_t)cpr;
            const dim3 grid((uint32_t)col_tiles, (uint32_t)steps);
#define CASE(TW_)                                                       \
    case TW_:                                                           \
        dropout_kernel<DT, TW_><<<grid, kDropThreads, 0, st>>>(d);      \
        break;
            switch (tw) {
                CASE(1) CASE(2) CASE(4) CASE(8) CASE(16) CASE(32) CASE(64)
            default:
                return NHP_ERR_SHAPE;
            }
#undef CASE
            return launch_result();
        }
    }
    const int64_t total = rows * cols;
    const int64_t blocks = (total + kDropThreads - 1) / kDropThreads;
    if (!grid_fits(blocks, kDropThreads)) return NHP_ERR_SHAPE;
    dropout_scalar_kernel<DT><<<(uint32_t)blocks, kDropThreads, 0, st>>>(d, (uint64_t)total, (uint64_t)cols);
    return launch_result();
}

static int dropout_entry(void* out, const void* a, const void* bias, const void* residual, int64_t rows, int64_t cols,
                         float p, uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    if (rows < 0 || cols < 0 || !(p >= 0.0f && p < 1.0f)) return NHP_ERR_SHAPE;
    if (rows > 0 && cols > ((int64_t)1 << 62) / rows) return NHP_ERR_SHAPE;
    if (rows == 0 || cols == 0) return NHP_OK;
    if (!out || !a) return NHP_ERR_NULL;
    DropArgs d{};
    d.out = out;
    d.a = a;
    d.residual = residual;
    d.bias = bias;
    const double keep = 1.0 - (double)p;
    uint32_t threshold = (uint32_t)(keep * 65536.0 + 0.5);
    d.threshold = threshold > 65536u ? 65536u : threshold;
    d.scale = (float)(1.0 / keep);
    d.seed_lo = (uint32_t)seed;
    d.seed_hi = (uint32_t)(seed >> 32);
    d.off_lo = (uint32_t)offset;
    d.off_hi = (uint32_t)(offset >> 32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case NHP_F16:
        return dropout_launch<NHP_F16>(d, rows, cols, st);
    case NHP_BF16:
        return dropout_launch<NHP_BF16>(d, rows, cols, st);
    default:
        return dropout_launch<NHP_F32>(d, rows, cols, st);
    }
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int nhp_bias_dropout_add(void* out, const void* x, const void* bias, const void* residual, int64_t rows,
                         int64_t cols, float p, uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    return dropout_entry(out, x, bias, residual, rows, cols, p, seed, offset, dtype, stream);
}

int nhp_dropout_bwd(void* dx, const void* g, int64_t rows, int64_t cols, float p, uint64_t seed, uint64_t offset,
                    int dtype, void* stream)
{
    return dropout_entry(dx, g, nullptr, nullptr, rows, cols, p, seed, offset, dtype, stream);
}

// The four output words of Philox4x32-10 for a counter and a key (host-visible for known-answer tests).
void nhp_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = counter[0], c1 = counter[1], c2 = counter[2], c3 = counter[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c0 = n0;
        c1 = (uint32_t)p1;
        c2 = n2;
        c3 = (uint32_t)p0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

}  // extern "C"
