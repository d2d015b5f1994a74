// Data-movement probes for gfx950: kernels that only move bytes, in the access patterns of the
// library's kernels, so that a kernel's time can be set against what the memory system gives for
// its pattern and size. Built into libneox_probe.so, which only bench.py loads; nothing of the
// library proper depends on it.
//
//   nhp_probe_copy            plain streaming copy, one 16-byte chunk per thread, no loop: the
//                             fastest copy shape measured on MI355X (more bytes per thread, grid-
//                             stride loops and XCD-contiguous orders are all slower)
//   nhp_probe_streams         n_in input streams (0..3) and one or no output stream of the same size, one
//                             16-byte chunk of each per thread: the traffic mix of the element-wise and
//                             normalisation backward kernels (two or three tensors in, one out) and of a
//                             pure reduction (one tensor in, nothing out)
//   nhp_probe_causal_pattern  the causal softmax forward's traffic: row q of every [n, n] matrix
//                             is read up to the 16-byte chunk that holds column q and written in
//                             full; two waves per row, two chunks per lane for n = 2048, as the
//                             forward kernel is launched
//   nhp_probe_causal_bwd_pattern  the causal softmax backward's traffic: the rows of two tensors read up to
//                             the diagonal, the first tensor's rows overwritten in full
//   nhp_probe_masked_pattern  the padding-mask softmax forward's traffic at [b, np, sq, 2048]: the mask row, the
//                             chunks of the scores that are not all padding, the whole row written
//   nhp_probe_seq_major_pattern  the traffic of the transposing rotary kernel: a [rows, 128, s]
//                             tensor (contiguous along s) is read in runs of 64 positions per
//                             feature and written as [s, rows, 128], whole 256-byte head vectors,
//                             through one 16-byte LDS store and load per chunk and one barrier;
//                             the data is not transposed (what arrives where is not the point)
//   nhp_probe_strided_runs    the traffic of the rotary kernels on q and k given as slices of one fused
//                             projection buffer [.., 3 * d]: runs of 2^k chunks that lie a fixed distance
//                             apart are read and written either to one contiguous output (one tensor per
//                             launch: 256 of every 768 bytes at d = 128) or, split in halves, to two
//                             contiguous outputs (q and k in one pass: 512 of every 768 bytes); two chunks
//                             per thread, all loads first, as rope_lean_kernel is launched

#include "common.hpp"

namespace nhp {

__global__ void __launch_bounds__(1024)
probe_copy_kernel(u32x4* out, const u32x4* in, size_t chunks)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < chunks) store16_stream(out + i, load16_stream(in + i));
}

// out = in0 ^ in1 ^ in2 (as many as given); without an output the value is only consumed.
template <int N_IN, bool WRITE>
__global__ void __launch_bounds__(256)
probe_streams_kernel(u32x4* out, const u32x4* in0, const u32x4* in1, const u32x4* in2, size_t chunks)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= chunks) return;
    // without inputs: index-dependent bits (what the bytes hold matters for the time, constants are faster)
    const uint32_t h = (uint32_t)i * 2654435761u;
    u32x4 v = u32x4{h, h ^ 0x9e3779b9u, h * 0x85ebca6bu, ~h};
    u32x4 a, b, c;
    if (N_IN > 0) a = load16_stream(in0 + i);
    if (N_IN > 1) b = load16_stream(in1 + i);
    if (N_IN > 2) c = load16_stream(in2 + i);
    if (N_IN > 0) v ^= a;
    if (N_IN > 1) v ^= b;
    if (N_IN > 2) v ^= c;
    if (WRITE) {
        store16_stream(out + i, v);
    } else if ((v[0] ^ v[1] ^ v[2] ^ v[3]) == 0x9e3779b9u && v[0] == 0x12345678u) {
        out[0] = v;  // practically never: keeps the loads alive
    }
}

// K chunks per lane, W waves per row (chunk c of a row belongs to (k, w, l) with c = (k*W + w)*64 + l,
// the softmax kernels' layout); workgroup = one row.
template <int K, int W>
__global__ void __launch_bounds__(W * 64)
probe_causal_pattern_kernel(uint16_t* y, const uint16_t* x, uint32_t n)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x;
    const uint32_t q = row % n;
    const int w = (int)((wave + blockIdx.x) % W);
    const uint16_t* xr = x + (size_t)row * n;
    uint16_t* yr = y + (size_t)row * n;
    u32x4 raw[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = (uint32_t)((k * W + w) * 64 + lane) * 8u;
        raw[k] = u32x4{0, 0, 0, 0};
        if (col < n && col <= q) raw[k] = load16_stream(xr + col);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = (uint32_t)((k * W + w) * 64 + lane) * 8u;
        if (col < n) store16_stream(yr + col, raw[k]);
    }
}

// The causal softmax backward's traffic: row q of every [n, n] matrix of g and of y is read up to the chunk
// that holds column q, and the row of g is overwritten in full (in place, as the library's backward works).
template <int K, int W>
__global__ void __launch_bounds__(W * 64)
probe_causal_bwd_pattern_kernel(uint16_t* g, const uint16_t* y, uint32_t n)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x;
    const uint32_t q = row % n;
    const int w = (int)((wave + blockIdx.x) % W);
    uint16_t* gr = g + (size_t)row * n;
    const uint16_t* yr = y + (size_t)row * n;
    u32x4 a[K], b[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = (uint32_t)((k * W + w) * 64 + lane) * 8u;
        a[k] = u32x4{0, 0, 0, 0};
        b[k] = u32x4{0, 0, 0, 0};
        if (col < n && col <= q) {
            a[k] = load16_stream(gr + col);
            b[k] = load16_stream(yr + col);
        }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = (uint32_t)((k * W + w) * 64 + lane) * 8u;
        if (col < n) store16_stream(gr + col, a[k] ^ b[k]);
    }
}

// The padding-mask softmax forward's traffic at 2048 keys: a workgroup of two waves takes one (batch entry,
// query) row for two heads: it reads the row's 2048 mask bytes, then for each head the 16-byte chunks of the
// scores whose 8 mask bytes are not all 1, and writes the whole row (two chunks per lane and wave, as the
// library's kernel is launched; workgroups ordered (batch entry, head pair, query)).
__global__ void __launch_bounds__(128)
probe_masked_pattern_kernel(uint16_t* y, const uint16_t* x, const uint8_t* mask, uint32_t sq, uint32_t np)
{
    constexpr uint32_t n = 2048;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t pairs = np / 2;
    const uint32_t id = blockIdx.x;
    const uint32_t bi = id / (pairs * sq);
    const uint32_t r = id - bi * pairs * sq;
    const uint32_t hp = r / sq, qi = r - hp * sq;
    const uint8_t* mrow = mask + ((size_t)bi * sq + qi) * n;
    bool live[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const uint32_t col = ((k * 2 + wave) * 64 + lane) * 8u;
        const u32x2 v = load8(mrow + col);
        live[k] = !(v[0] == 0x01010101u && v[1] == 0x01010101u);
    }
    for (uint32_t h = hp * 2; h < hp * 2 + 2; ++h) {
        const size_t base = (((size_t)bi * np + h) * sq + qi) * n;
        u32x4 raw[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint32_t col = ((k * 2 + wave) * 64 + lane) * 8u;
            raw[k] = u32x4{0, 0, 0, 0};
            if (live[k]) raw[k] = load16_stream(x + base + col);
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint32_t col = ((k * 2 + wave) * 64 + lane) * 8u;
            store16_stream(y + base + col, raw[k]);
        }
    }
}

// One workgroup per (row, 64 positions): thread t loads 16 bytes (8 positions) of features
// (t >> 3) + 32 p, p = 0..3, stages them in LDS, and stores the tile as 64 head vectors of 256 bytes.
__global__ void __launch_bounds__(256)
probe_seq_major_kernel(uint16_t* out, const uint16_t* in, uint32_t rows, uint32_t s)
{
    __shared__ u32x4 tile[64 * 16];
    const uint32_t tid = threadIdx.x;
    const uint32_t r = blockIdx.x;
    const uint32_t s0 = blockIdx.y * 64u;
    const uint32_t sc = tid & 7u, dr = tid >> 3;
    u32x4 raw[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) raw[p] = load16_stream(in + ((size_t)r * 128u + p * 32u + dr) * s + s0 + sc * 8u);
#pragma unroll
    for (int p = 0; p < 4; ++p) tile[(p * 256u + tid) ^ ((tid >> 4) & 7u)] = raw[p];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t idx = i * 256u + tid;
        const uint32_t row = idx >> 4, c = idx & 15u;
        store16_stream(out + ((size_t)(s0 + row) * rows + r) * 128u + c * 8u, tile[idx ^ (row & 7u)]);
    }
}

// Run r holds chunks [r * stride, r * stride + 2^LOG_RUN). SPLIT: the first half of every run goes to out0,
// the second to out1 (each contiguous); otherwise the whole run to out0.
template <int LOG_RUN, bool SPLIT>
__global__ void __launch_bounds__(256)
probe_strided_runs_kernel(u32x4* out0, u32x4* out1, const u32x4* in, uint32_t runs, uint32_t stride)
{
    constexpr uint32_t RUN = 1u << LOG_RUN, HALF = RUN / 2;
    const uint32_t i0 = blockIdx.x * 512u + threadIdx.x;
    u32x4 raw[2];
    bool on[2];
    size_t dst[2];
    bool second[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t i = i0 + u * 256u;
        const uint32_t r = i >> LOG_RUN, c = i & (RUN - 1);
        on[u] = r < runs;
        const uint32_t rr = on[u] ? r : runs - 1;
        raw[u] = load16_stream(in + (size_t)rr * stride + c);
        second[u] = SPLIT && c >= HALF;
        dst[u] = SPLIT ? (size_t)rr * HALF + (c & (HALF - 1)) : (size_t)rr * RUN + c;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
        if (on[u]) store16_stream((second[u] ? out1 : out0) + dst[u], raw[u]);
}

}  // namespace nhp

using namespace nhp;

extern "C" {

// `runs` runs of `run_chunks` (16 or 32) 16-byte chunks, `stride_chunks` apart in `in`. split = 0: copied to out0
// back to back; split = 1: first halves to out0, second halves to out1.
int nhp_probe_strided_runs(void* out0, void* out1, const void* in, int64_t runs, int run_chunks, int64_t stride_chunks,
                           int split, void* stream)
{
    if (runs < 1 || (run_chunks != 16 && run_chunks != 32) || stride_chunks < run_chunks ||
        stride_chunks >= ((int64_t)1 << 31) || runs * run_chunks >= ((int64_t)1 << 31))
        return NHP_ERR_SHAPE;
    if (!out0 || !in || (split && !out1)) return NHP_ERR_NULL;
    const int64_t blocks = (runs * run_chunks + 511) / 512;
    if (!grid_fits(blocks, 256)) return NHP_ERR_SHAPE;
    launch_prepare();
    hipStream_t st = static_cast<hipStream_t>(stream);
    u32x4* o0 = static_cast<u32x4*>(out0);
    u32x4* o1 = static_cast<u32x4*>(out1);
    const u32x4* ip = static_cast<const u32x4*>(in);
    if (run_chunks == 16 && !split)
        probe_strided_runs_kernel<4, false><<<(uint32_t)blocks, 256, 0, st>>>(o0, o1, ip, (uint32_t)runs, (uint32_t)stride_chunks);
    else if (run_chunks == 32 && split)
        probe_strided_runs_kernel<5, true><<<(uint32_t)blocks, 256, 0, st>>>(o0, o1, ip, (uint32_t)runs, (uint32_t)stride_chunks);
    else if (run_chunks == 32)
        probe_strided_runs_kernel<5, false><<<(uint32_t)blocks, 256, 0, st>>>(o0, o1, ip, (uint32_t)runs, (uint32_t)stride_chunks);
    else
        probe_strided_runs_kernel<4, true><<<(uint32_t)blocks, 256, 0, st>>>(o0, o1, ip, (uint32_t)runs, (uint32_t)stride_chunks);
    return launch_result();
}

// Copies `bytes` (a multiple of 16) from in to out with workgroups of `threads` (64..1024) threads.
int nhp_probe_copy(void* out, const void* in, int64_t bytes, int threads, void* stream)
{
    if (bytes < 0 || bytes % 16 != 0 || threads < 64 || threads > 1024 || threads % 64 != 0) return NHP_ERR_SHAPE;
    if (bytes == 0) return NHP_OK;
    if (!out || !in) return NHP_ERR_NULL;
    const int64_t chunks = bytes / 16;
    const int64_t blocks = (chunks + threads - 1) / threads;
    if (!grid_fits(blocks, threads)) return NHP_ERR_SHAPE;
    launch_prepare();
    probe_copy_kernel<<<(uint32_t)blocks, threads, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4*>(out), static_cast<const u32x4*>(in), (size_t)chunks);
    return launch_result();
}

// `bytes` (a multiple of 16) per stream; n_in = 0..3 inputs, with_out = 1: one output of that size, 0: none
// (out must still point to at least 16 writable bytes).
int nhp_probe_streams(void* out, const void* in0, const void* in1, const void* in2, int64_t bytes, int n_in,
                      int with_out, void* stream)
{
    if (bytes < 0 || bytes % 16 != 0 || n_in < 0 || n_in > 3 || (n_in == 0 && !with_out)) return NHP_ERR_SHAPE;
    if (bytes == 0) return NHP_OK;
    if (!out || (n_in > 0 && !in0) || (n_in > 1 && !in1) || (n_in > 2 && !in2)) return NHP_ERR_NULL;
    const int64_t chunks = bytes / 16;
    const int64_t blocks = (chunks + 255) / 256;
    if (!grid_fits(blocks, 256)) return NHP_ERR_SHAPE;
    launch_prepare();
    hipStream_t st = static_cast<hipStream_t>(stream);
    u32x4* o = static_cast<u32x4*>(out);
    const u32x4* a = static_cast<const u32x4*>(in0);
    const u32x4* b = static_cast<const u32x4*>(in1);
    const u32x4* c = static_cast<const u32x4*>(in2);
#define NHP_PROBE_CASE(N_, W_)                                                                           \
    if (n_in == N_ && (with_out != 0) == W_) {                                                           \
        probe_streams_kernel<N_, W_><<<(uint32_t)blocks, 256, 0, st>>>(o, a, b, c, (size_t)chunks);      \
        return launch_result();                                                                          \
    }
    NHP_PROBE_CASE(0, true) NHP_PROBE_CASE(1, true) NHP_PROBE_CASE(2, true) NHP_PROBE_CASE(3, true)
    NHP_PROBE_CASE(1, false) NHP_PROBE_CASE(2, false) NHP_PROBE_CASE(3, false)
#undef NHP_PROBE_CASE
    return NHP_ERR_SHAPE;
}

// y, x: [batches, n, n] 16-bit elements, n = 2048 (two waves of two chunks per lane) or 8192
// (eight waves of two chunks per lane).
int nhp_probe_causal_pattern(void* y, const void* x, int64_t batches, int64_t n, void* stream)
{
    if (batches < 1 || (n != 2048 && n != 8192) || batches * n >= ((int64_t)1 << 31)) return NHP_ERR_SHAPE;
    if (!y || !x) return NHP_ERR_NULL;
    launch_prepare();
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t rows = (uint32_t)(batches * n);
    if (n == 2048)
        probe_causal_pattern_kernel<2, 2><<<rows, 128, 0, st>>>(static_cast<uint16_t*>(y), static_cast<const uint16_t*>(x), 2048u);
    else
        probe_causal_pattern_kernel<2, 8><<<rows, 512, 0, st>>>(static_cast<uint16_t*>(y), static_cast<const uint16_t*>(x), 8192u);
    return launch_result();
}

// g (overwritten), y: [batches, n, n] 16-bit elements, n = 2048 (two waves of two chunks per lane) or 8192 (eight waves).
int nhp_probe_causal_bwd_pattern(void* g, const void* y, int64_t batches, int64_t n, void* stream)
{
    if (batches < 1 || (n != 2048 && n != 8192) || batches * n >= ((int64_t)1 << 31)) return NHP_ERR_SHAPE;
    if (!g || !y) return NHP_ERR_NULL;
    launch_prepare();
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t rows = (uint32_t)(batches * n);
    if (n == 2048)
        probe_causal_bwd_pattern_kernel<2, 2><<<rows, 128, 0, st>>>(static_cast<uint16_t*>(g), static_cast<const uint16_t*>(y), 2048u);
    else
        probe_causal_bwd_pattern_kernel<2, 8><<<rows, 512, 0, st>>>(static_cast<uint16_t*>(g), static_cast<const uint16_t*>(y), 8192u);
    return launch_result();
}

// y, x: [b, np, sq, 2048] 16-bit elements, mask: [b, 1, sq, 2048] bytes (1 = masked); np even.
int nhp_probe_masked_pattern(void* y, const void* x, const void* mask, int64_t b, int64_t np, int64_t sq, void* stream)
{
    if (b < 1 || np < 2 || np % 2 != 0 || sq < 1 || b * (np / 2) * sq >= ((int64_t)1 << 31)) return NHP_ERR_SHAPE;
    if (!y || !x || !mask) return NHP_ERR_NULL;
    launch_prepare();
    probe_masked_pattern_kernel<<<(uint32_t)(b * (np / 2) * sq), 128, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint16_t*>(y), static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(mask), (uint32_t)sq,
        (uint32_t)np);
    return launch_result();
}

// in: [rows, 128, s], out: [s, rows, 128], 16-bit elements; s a multiple of 64.
int nhp_probe_seq_major_pattern(void* out, const void* in, int64_t rows, int64_t s, void* stream)
{
    if (rows < 1 || s < 64 || s % 64 != 0 || s / 64 > 65535 || rows >= ((int64_t)1 << 24)) return NHP_ERR_SHAPE;
    if (!out || !in) return NHP_ERR_NULL;
    launch_prepare();
    probe_seq_major_kernel<<<dim3((uint32_t)rows, (uint32_t)(s / 64)), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint16_t*>(out), static_cast<const uint16_t*>(in), (uint32_t)rows, (uint32_t)s);
    return launch_result();
}

}  // extern "C"
