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
//   n <= 512        : L = n/8 rounded up to a power of two, K = 1, 64/L rows per wave
//   n <= 65536      : W = 1..8 (16 beyond 32768) waves per row with K = 1..8
//                     chunks per lane; partial max / sum are exchanged through
//                     2*W floats of LDS (see plan_row for the choice)
//   otherwise, or if n % 8 != 0 or a pointer is not 16-byte aligned:
//                     a scalar three-pass kernel (one workgroup per row).
//
// Arithmetic (fp32): z = x*scale, m = max z, e = 2^((z-m)*log2(e) + 64),
// p = e * (1 / sum e). The constant 64 scales every e of a row by 2^64, which
// cancels in p, and keeps e out of the range where v_exp_f32 flushes to zero
// down to 2^-190, so probabilities in the bf16 subnormal range are still produced.
//
// Masks are applied by index: in the causal kernels only the columns of the
// band max(0, q - window) <= k <= q are loaded (window = none: 0 <= k <= q),
// everything else is written as zeros; the band also ends at the number of
// real keys of the row's batch entry when key lengths are given; an AliBi bias
// is computed from (q - k) and the head's slope, an additive bias tensor is
// read beside the scores; in the padding-mask kernel a chunk whose 8 mask
// bytes are all 1 is not loaded.
//
// Attention dropout: the forward also writes dropout(y), the
// backward first applies the dropout backward to dy; the keep mask is
// regenerated from a counter-based generator, never stored.

#include "common.hpp"

namespace nhp {

constexpr float kExpBias = 64.0f;
constexpr float kMaskFill = -10000.0f;  // scaled_masked_softmax.h:180-184 of the reference
// Row blocks of one head that are taken for every batch entry in turn when a bias tensor is shared by the
// batch (batch_interleaved_block); 0: all row blocks of a matrix.
constexpr int kBiasShareGroup = 0;

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
// `act`: bit k set = slot k holds at least one finite value (wave-uniform).
//
// With several waves per row every wave first reduces its own part against its
// own maximum m_w, then the (m_w, s_w) pairs are exchanged through LDS once:
//   M = max m_w,  S = sum s_w * 2^((m_w - M) log2 e),  p = e * 2^((m_w - M) log2 e) / S
// which needs one barrier instead of one for the maximum and one for the sum.
template <int L, int K, int W>
__device__ __forceinline__ void softmax_tile(float (&z)[K][8], uint32_t act, float* lds, int wave, int lane)
{
    float m = kNegInf;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (act >> k & 1u) {
#pragma unroll
            for (int j = 0; j < 8; ++j) m = fmaxf(m, z[k][j]);
        }
    }
    m = group_reduce<OpMax, L>(m);

    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (act >> k & 1u) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float e = exp2_raw(fmaf(z[k][j] - m, kLog2e, kExpBias));
                z[k][j] = e;
                sum += e;
            }
        }
    }
    sum = group_reduce<OpSum, L>(sum);

    float inv;
    if constexpr (W == 1) {
        inv = 1.0f / sum;
    } else {
        if (lane == 0) {
            lds[wave] = m;
            lds[16 + wave] = sum;
        }
        __syncthreads();
        float big = lds[0];
#pragma unroll
        for (int i = 1; i < W; ++i) big = fmaxf(big, lds[i]);
        float total = 0.0f;
#pragma unroll
        for (int i = 0; i < W; ++i) total = fmaf(lds[16 + i], exp2_raw((lds[i] - big) * kLog2e), total);
        // a wave without any valid column has m = -inf and never uses inv
        inv = exp2_raw((m - big) * kLog2e) / total;
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (act >> k & 1u) {
#pragma unroll
            for (int j = 0; j < 8; ++j) z[k][j] *= inv;
        }
    }
}

// Locate the row this lane works on. Rows are numbered over the whole tensor;
// `q` is the row's index inside its [n_q, n] matrix and `mat` that matrix.
template <typename G>
__device__ __forceinline__ void locate_row(uint32_t block, uint32_t rows_per_matrix, int wave, int lane,
                                           int lanes_per_row, uint32_t& row, uint32_t& q, uint32_t& mat)
{
    const uint32_t row0 = block * (uint32_t)G::kRowsPerBlock;
    mat = row0 / rows_per_matrix;  // scalar: depends on the block id only
    const uint32_t q0 = row0 - mat * rows_per_matrix;
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
    while (q >= rows_per_matrix) {
        q -= rows_per_matrix;
        ++mat;
    }
}

// Workgroup order for a bias tensor [heads, n_q, n] that the `batch` entries of the batch share. In
// row-major order the matrices that share a head's bias are a whole batch entry apart and every one of
// them fetches that bias from HBM again. Here `group` consecutive row blocks of one head are taken for every
// batch entry in turn (group * batch workgroups), then the head's next row blocks: workgroup id -> block
// number of the row-major order. The library uses group = all row blocks of a matrix, i.e. the matrices
// in the order (head, batch entry): the batch entries of a head then follow each other, each XCD sees the
// same eighth of the bias rows again one matrix later and finds them in its L2 (2048 keys: 1 MiB per XCD
// and head; the scores pass through with streaming hints), which took the fetched bytes from 1.8 x to
// 1.03 x the algorithmic ones at [8 * 16, 2048, 2048] and 0-2 % off the time. Smaller groups save the same
// bytes but interleave the DRAM streams of `batch` matrices and cost 10 % (groups of 8 or 64 blocks).
__device__ __forceinline__ uint32_t batch_interleaved_block(uint32_t id, uint32_t blocks_per_matrix, uint32_t heads,
                                                            uint32_t batch, uint32_t group)
{
    const uint32_t span = group * batch;
    const uint32_t g = id / span;  // (head, row-block group), head-major
    const uint32_t t = id - g * span;
    const uint32_t j = t / group, r = t - j * group;
    const uint32_t groups_per_matrix = blocks_per_matrix / group;
    const uint32_t head = g / groups_per_matrix;
    const uint32_t qg = g - head * groups_per_matrix;
    return (j * heads + head) * blocks_per_matrix + qg * group + r;
}

// The columns of row q that take part in a causal softmax: [lo, hi) with
// hi = min(q + 1, limit) and lo = max(0, q - window) (window = 0xffffffff: no
// lower bound; limit = the number of real keys of the row's batch entry).
// hi <= lo is an empty band (possible with key lengths only): the forward writes 1/n in every
// column of such a row, the backward zeros.
struct Band {
    uint32_t lo, hi;
};
__device__ __forceinline__ Band causal_band(uint32_t q, uint32_t window, bool ok, uint32_t limit = 0xffffffffu)
{
    Band b;
    b.hi = ok ? min(q + 1, limit) : 0;
    b.lo = (ok && q > window) ? q - window : 0;
    if (b.hi <= b.lo) b.hi = b.lo = 0;  // one form for the empty band: no chunk straddles it
    return b;
}

// Columns [lo, hi) of row q that have to hold a value when the caller only consumes the result in square
// blocks of 2^zshift rows and columns: from the start of the block that holds the first key visible to the
// first row of q's block (column 0 without a window) to the end of the block that holds the diagonal.
// zshift == 0: the whole row.
__device__ __forceinline__ Band written_range(uint32_t q, uint32_t window, uint32_t n, uint32_t zshift)
{
    Band b;
    b.lo = 0;
    b.hi = n;
    if (zshift != 0) {
        b.hi = min(n, ((q >> zshift) + 1u) << zshift);
        const uint32_t r0 = (q >> zshift) << zshift;
        b.lo = r0 > window ? ((r0 - window) >> zshift) << zshift : 0u;
    }
    return b;
}

// Number of real keys of matrix `mat` ([batch * heads] matrices, one length per batch entry).
__device__ __forceinline__ uint32_t key_limit(const int32_t* key_lengths, uint32_t mat, uint32_t heads)
{
    if (key_lengths == nullptr) return 0xffffffffu;
    const int32_t len = key_lengths[mat / heads];
    return len < 0 ? 0u : (uint32_t)len;
}

// Bit k set: register slot k of wave-slot w holds at least one column of the
// band. Wave-uniform for full-wave rows; all K bits for rows sharing a wave.
template <int L, int K, int W>
__device__ __forceinline__ uint32_t active_slots(const Band& band, int w)
{
    if constexpr (L == 64) {
        uint32_t act = 0;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t start = (uint32_t)(k * W + w) * 512u;
            if (start < band.hi && start + 512u > band.lo) act |= 1u << k;
        }
        return act;
    } else {
        return (1u << K) - 1u;
    }
}

// ---------------------------------------------------------------------------
// Causal forward
// ---------------------------------------------------------------------------
// EXTRA selects what is compiled in besides the plain kernel (which keeps its
// registers for loads in flight): kPerHead = bias tensor, AliBi, key lengths;
// kDropout = a second output `dropped` = dropout(y) (y, the probabilities, is
// still written: the backward needs it).
enum CausalExtra { kPlain = 0, kPerHead = 1, kDropout = 2, kPerHeadDropout = 3 };  // bit flags

template <int DT, int L, int K, int W, int BW, int EXTRA>
__global__ void __launch_bounds__((Geo<L, K, W, BW>::kThreads))
causal_fwd_kernel(uint16_t* y, const uint16_t* x, float scale, uint32_t total_rows, uint32_t n, uint32_t window,
                  const float* slopes, const uint16_t* bias, const int32_t* key_lengths, uint32_t heads,
                  uint16_t* dropped, DropoutKey dk, uint32_t zshift, uint32_t share_batch, uint32_t share_group)
{
    using G = Geo<L, K, W, BW>;
    constexpr bool PER_HEAD = (EXTRA & kPerHead) != 0;
    constexpr bool DROPOUT = (EXTRA & kDropout) != 0;
    __shared__ float lds[32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & (L - 1);
    // Which of the row's W interleaved segment sets this wave takes rotates with
    // the row: the leftmost segments are the ones most often below the diagonal,
    // and wave i of every workgroup sits on the same SIMD of its CU.
    const int w = (W > 1) ? (int)((wave + blockIdx.x) % W) : 0;

    // share_batch > 1 (only with a bias tensor): the batch entries of a head follow each other
    uint32_t block = blockIdx.x;
    if (PER_HEAD && share_batch > 1)
        block = batch_interleaved_block(block, n / (uint32_t)G::kRowsPerBlock, heads, share_batch, share_group);
    uint32_t row, q, mat;
    locate_row<G>(block, n, wave, lane, L, row, q, mat);
    const bool ok = row < total_rows;
    // columns [lo, hi) take part
    const Band band = causal_band(q, window, ok, (PER_HEAD && ok) ? key_limit(key_lengths, mat, heads) : 0xffffffffu);

    const uint16_t* xr = x + (size_t)row * n;
    uint16_t* yr = y + (size_t)row * n;

    const uint32_t act = active_slots<L, K, W>(band, w);

    u32x4 raw[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        raw[k] = u32x4{0, 0, 0, 0};
        if ((act >> k & 1u) && col < band.hi && col + 8 > band.lo) raw[k] = load16_stream(xr + col);
    }

    // Additive bias [heads, n, n] (e.g. a relative-position bias shared by the batch):
    // added to the score in the storage dtype, as `scores += bias` does in eager torch.
    if (PER_HEAD && bias != nullptr) {
        const uint16_t* br = bias + ((size_t)(mat % heads) * n + q) * n;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t col = chunk_col<L, W>(k, w, l);
            if ((act >> k & 1u) && col < band.hi && col + 8 > band.lo) {
                const u32x4 rb = load16(br + col);  // re-used by every batch entry: keep it cacheable
                float f[8], g[8];
                unpack8<DT>(raw[k], f);
                unpack8<DT>(rb, g);
#pragma unroll
                for (int j = 0; j < 8; ++j) f[j] = f[j] + g[j];
                raw[k] = pack8<DT>(f);
            }
        }
    }

    // AliBi: bias[q][k] = (-(q - k)) * slope in the storage dtype, added to the
    // score in the storage dtype (what `scores + alibi_matrix` does in eager torch)
    const bool alibi = PER_HEAD && slopes != nullptr;
    float slope = 0.0f;
    if (alibi) slope = Half2<DT>::round(slopes[mat % heads]);

    float z[K][8];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (act >> k & 1u) {
            const uint32_t col = chunk_col<L, W>(k, w, l);
            float f[8];
            unpack8<DT>(raw[k], f);
            if (alibi) {
                // -(q - k) from the chunk's first column; every rounding takes two elements at a time
                const float d0 = (float)((int)col - (int)q);
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    float da = d0 + (float)j, db = d0 + (float)(j + 1);
                    round_pair<DT>(da, db);
                    float pa = da * slope, pb = db * slope;
                    round_pair<DT>(pa, pb);
                    f[j] = f[j] + pa;
                    f[j + 1] = f[j + 1] + pb;
                    round_pair<DT>(f[j], f[j + 1]);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) z[k][j] = f[j] * scale;
            // only slots that straddle an end of the band need masking
            bool edge;
            if constexpr (G::kUniformRow) {
                const uint32_t start = (uint32_t)(k * W + w) * 512u;
                edge = start + 512u > band.hi || start < band.lo;
            } else {
                edge = true;
            }
            if (edge) {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    z[k][j] = (col + j < band.hi && col + j >= band.lo) ? z[k][j] : kNegInf;
            }
        }
    }

    softmax_tile<L, K, W>(z, act, lds, wave, lane);

    // The whole row is written in one go, zeros outside the band included (as far as the caller reads
    // them): splitting a row's stores in time costs DRAM efficiency.
    const Band wr = written_range(q, window, n, zshift);
    // A row that the key lengths leave without any key: 1/n in every column, what the softmax over a
    // row of equal fill values gives on the reference's torch branch (megatron/model/fused_softmax.py:184-199).
    uint32_t fill = 0;
    if constexpr (PER_HEAD) {
        if (ok && band.hi == 0) fill = Half2<DT>::pack(1.0f / (float)n, 1.0f / (float)n);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        if (ok && col < wr.hi && col >= wr.lo) {
            if (PER_HEAD && fill != 0) {
                store16_stream(yr + col, u32x4{fill, fill, fill, fill});
                if constexpr (DROPOUT) {
                    const float v = Half2<DT>::lo(fill);
                    float f[8];
                    const Philox rnd = dropout_bits(dk, (uint64_t)row * n + col);
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[j] = random16(rnd, j) < dk.threshold ? v * dk.scale : 0.0f;
                    store16_stream(dropped + (size_t)row * n + col, pack8<DT>(f));
                }
            } else if ((act >> k & 1u) && col < band.hi && col + 8 > band.lo) {
                const u32x4 py = pack8<DT>(z[k]);
                store16_stream(yr + col, py);
                if constexpr (DROPOUT) {
                    // dropout of the stored (rounded) probabilities, as the separate dropout kernel would see them
                    float f[8];
                    unpack8<DT>(py, f);
                    const Philox rnd = dropout_bits(dk, (uint64_t)row * n + col);
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[j] = random16(rnd, j) < dk.threshold ? f[j] * dk.scale : 0.0f;
                    store16_stream(dropped + (size_t)row * n + col, pack8<DT>(f));
                }
            } else {
                store16_stream(yr + col, u32x4{0, 0, 0, 0});
                if constexpr (DROPOUT) store16_stream(dropped + (size_t)row * n + col, u32x4{0, 0, 0, 0});
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Causal forward for rows of at most 64 chunks (512 keys), plain variant. One chunk per lane
// covers such a row, and half of the chunks are above the diagonal and never loaded: a wave
// of the general kernel has a few hundred bytes in flight. Here a lane takes the same chunk
// of R rows (64 / L rows apart), all loads issued first; every row is reduced on its own with
// the arithmetic of softmax_tile, so the results are the same bits. Measured at 1 GiB of
// scores: 53 -> 63 % of the HBM peak at 256 keys, 62 -> 65 % at 512 (eight rows in flight, or
// four chunks per lane with masked slots skipped by the whole wave, gain nothing more).
// ---------------------------------------------------------------------------
constexpr int kShortRows = 4;  // rows in flight per lane (8 measured slower)

template <int DT, int L, int R>
__global__ void __launch_bounds__(256)
causal_fwd_short_kernel(uint16_t* y, const uint16_t* x, float scale, uint32_t total_rows, uint32_t n, uint32_t window)
{
    constexpr int RPW = kWave / L;  // rows per wave and step
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l = lane & (L - 1);
    const uint32_t col = (uint32_t)l * 8u;
    const uint32_t row0 = (blockIdx.x * 4u + (uint32_t)wave) * (uint32_t)(RPW * R) + (uint32_t)(lane / L);
    uint32_t q = row0 % n;

    u32x4 raw[R];
    Band band[R];
    bool ok[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const uint32_t row = row0 + (uint32_t)(i * RPW);
        ok[i] = row < total_rows && col < n;
        band[i] = causal_band(q, window, ok[i]);
        raw[i] = u32x4{0, 0, 0, 0};
        if (col < band[i].hi && col + 8 > band[i].lo) raw[i] = load16_stream(x + (size_t)row * n + col);
        q += RPW;
        while (q >= n) q -= n;
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        float z[8];
        unpack8<DT>(raw[i], z);
        float m = kNegInf;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            z[j] = (col + j < band[i].hi && col + j >= band[i].lo) ? z[j] * scale : kNegInf;
            m = fmaxf(m, z[j]);
        }
        m = group_reduce<OpMax, L>(m);
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            z[j] = exp2_raw(fmaf(z[j] - m, kLog2e, kExpBias));
            sum += z[j];
        }
        sum = group_reduce<OpSum, L>(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int j = 0; j < 8; ++j) z[j] *= inv;
        // lanes of rows beyond the tensor hold m = -inf and NaNs: not stored
        if (ok[i]) store16_stream(y + (size_t)(row0 + (uint32_t)(i * RPW)) * n + col, pack8<DT>(z));
    }
}

// ---------------------------------------------------------------------------
// Padding-mask forward. A wave owns the rows (b, q) of its lanes and walks
// over `heads_per_wave` heads with them, so the mask bytes of a row are
// fetched and decoded once per head group.
// ---------------------------------------------------------------------------
// DROP: also write dropped = dropout(y), as the causal kernel does.
// PER_HEAD: what the caller of the reference adds to the scores, or folds into the mask, before this
// softmax (megatron/model/transformer.py:580-588), done here instead of in passes of their own:
//   bias [np, sq, n] in the scores' dtype (attention_scores += rpe): added in the storage dtype;
//   AliBi slopes [np] (sq == n): the bias -(q - k) * slope for k <= q, nothing above the diagonal, with
//     the roundings of AliBi.forward (megatron/model/positional_embeddings.py:219-257);
//   key_lengths [b]: keys k >= key_lengths[b] count as masked (as if their mask bytes were 1).
template <int DT, int L, int K, int W, int BW, bool DROP, bool PER_HEAD>
__global__ void __launch_bounds__((Geo<L, K, W, BW>::kThreads))
masked_fwd_kernel(uint16_t* y, const uint16_t* x, const uint8_t* mask, float scale,
                  uint32_t bq_rows, uint32_t sq, uint32_t np, uint32_t n,
                  uint32_t heads_per_wave, uint32_t head_groups, int mask_per_batch, uint32_t row_blocks,
                  uint32_t tile, uint16_t* dropped, DropoutKey dk, const float* slopes, const uint16_t* bias,
                  const int32_t* key_lengths, uint32_t share_batch, uint32_t share_group)
{
    using G = Geo<L, K, W, BW>;
    __shared__ float lds[2][32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & (L - 1);
    const int w = (W > 1) ? wave : 0;

    // Workgroup order: `tile` consecutive row blocks (all query rows of a
    // sequence), then the next head group on the same rows, then the next tile.
    // Neighbouring workgroups thus work on consecutive score rows (what HBM
    // likes best), and a mask row is used again one tile later, from L2.
    // With a bias tensor shared by `share_batch` batch entries (a tile is then exactly one batch entry's
    // row blocks): `share_group` row blocks of one head group for every batch entry in turn, so that the
    // matrices sharing a bias follow each other (see batch_interleaved_block).
    const uint32_t id = blockIdx.x;
    uint32_t hg, rb;
    if (PER_HEAD && share_batch > 1) {
        const uint32_t flat = batch_interleaved_block(id, tile, head_groups, share_batch, share_group);
        const uint32_t m = flat / tile;  // batch entry * head_groups + head group
        const uint32_t bi_ = m / head_groups;
        hg = m - bi_ * head_groups;
        rb = bi_ * tile + (flat - m * tile);
    } else {
        const uint32_t per_tile = tile * head_groups;
        const uint32_t t = id / per_tile;
        const uint32_t r = id - t * per_tile;
        const uint32_t tile_rows = (t * tile + tile <= row_blocks) ? tile : row_blocks - t * tile;
        hg = r / tile_rows;
        rb = t * tile + (r - hg * tile_rows);
    }

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
    bool live[K];  // chunk inside the row with at least one unmasked column: scores are read
    bool dead[K];  // chunk inside the row with all eight columns masked: scores are not needed
    bool any_dead = false;
    uint32_t mb[K][2];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        const bool inb = ok && col < n;
        mb[k][0] = 0;
        mb[k][1] = 0;
        if (inb) {
            const u32x2 v = load8(mrow + col);
            mb[k][0] = v[0];
            mb[k][1] = v[1];
            if (PER_HEAD && key_lengths != nullptr) {
                // bytes of the keys at or beyond the sequence's length become 1
                const int32_t len = key_lengths[bi];
                const uint32_t limit = len < 0 ? 0u : (uint32_t)len;
                const uint32_t valid = limit > col ? limit - col : 0u;  // leading keys of the chunk that are real
                if (valid < 8u) {
                    const uint64_t beyond = ~(uint64_t)0 << (8u * valid);
                    const uint64_t bytes = ((((uint64_t)mb[k][1] << 32) | mb[k][0]) & ~beyond) | (0x0101010101010101ull & beyond);
                    mb[k][0] = (uint32_t)bytes;
                    mb[k][1] = (uint32_t)(bytes >> 32);
                }
            }
        }
        dead[k] = inb && (mb[k][0] == 0x01010101u) && (mb[k][1] == 0x01010101u);
        live[k] = inb && !dead[k];
        any_dead = any_dead || dead[k];
    }
    // Slots in which no lane of the wave has a masked key among its live columns skip the per-element
    // selection below (most slots: a padding mask has one ragged chunk per row, a causal one per slot row).
    bool mixed[K];
#pragma unroll
    for (int k = 0; k < K; ++k)
        mixed[k] = __builtin_amdgcn_ballot_w64(live[k] && (mb[k][0] | mb[k][1]) != 0u) != 0ull;

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
            if (live[k]) raw[k] = load16_stream(xr + col);
        }
        // the bias chunks are requested with the scores; both are used in the logit loop below
        u32x4 rbias[PER_HEAD ? K : 1];
        float slope = 0.0f;
        if constexpr (PER_HEAD) {
            if (bias != nullptr) {
                const uint16_t* br = bias + ((size_t)h * sq + qi) * n;
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    rbias[k] = u32x4{0, 0, 0, 0};
                    if (live[k]) rbias[k] = load16(br + chunk_col<L, W>(k, w, l));  // re-used by every batch entry
                }
            }
            if (slopes != nullptr) slope = Half2<DT>::round(slopes[h]);
        }

        // Chunks whose eight columns are all masked hold eight copies of the fill value:
        // they enter the maximum once, and share one exponential and one output value.
        float z[K][8];
        float m = any_dead ? kMaskFill : kNegInf;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (live[k]) {
                float f[8];
                unpack8<DT>(raw[k], f);
                if constexpr (PER_HEAD) {
                    if (bias != nullptr) {
                        float g[8];
                        unpack8<DT>(rbias[k], g);
#pragma unroll
                        for (int j = 0; j < 8; j += 2) {
                            f[j] = f[j] + g[j];
                            f[j + 1] = f[j + 1] + g[j + 1];
                            round_pair<DT>(f[j], f[j + 1]);
                        }
                    }
                    const uint32_t col = chunk_col<L, W>(k, w, l);
                    if (slopes != nullptr && col <= qi) {
                        // -(q - k) for the chunk's first column; formed anew for every head (an opaque value)
                        // so that the 8 K distances are not kept in registers across the loop over the heads
                        // Above the diagonal the AliBi matrix is 0: the distance is clamped there, which
                        // leaves the score as it is (a -0 becomes +0, the same logit).
                        float d0 = (float)((int)col - (int)qi);
                        asm volatile("" : "+v"(d0));
#pragma unroll
                        for (int j = 0; j < 8; j += 2) {
                            float da = fminf(d0 + (float)j, 0.0f), db = fminf(d0 + (float)(j + 1), 0.0f);
                            round_pair<DT>(da, db);
                            float pa = da * slope, pb = db * slope;
                            round_pair<DT>(pa, pb);
                            f[j] = f[j] + pa;
                            f[j + 1] = f[j + 1] + pb;
                            round_pair<DT>(f[j], f[j + 1]);
                        }
                    }
                }
                if (mixed[k]) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t byte = (mb[k][j >> 2] >> (8 * (j & 3))) & 0xffu;
                        z[k][j] = (byte == 1u) ? kMaskFill : f[j] * scale;
                        m = fmaxf(m, z[k][j]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        z[k][j] = f[j] * scale;
                        m = fmaxf(m, z[k][j]);
                    }
                }
            }
        }
        m = group_reduce<OpMax, L>(m);
        m = block_combine<OpMax, W>(m, lds[h & 1], wave, lane);

        const float e_dead = exp2_raw(fmaf(kMaskFill - m, kLog2e, kExpBias));
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (live[k]) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float e = exp2_raw(fmaf(z[k][j] - m, kLog2e, kExpBias));
                    z[k][j] = e;
                    sum += e;
                }
            } else if (dead[k]) {
                sum += 8.0f * e_dead;
            }
        }
        sum = group_reduce<OpSum, L>(sum);
        sum = block_combine<OpSum, W>(sum, lds[h & 1] + 16, wave, lane);
        const float inv = 1.0f / sum;
        const uint32_t pd = Half2<DT>::pack(e_dead * inv, e_dead * inv);

#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t col = chunk_col<L, W>(k, w, l);
            if (live[k]) {
                float o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = z[k][j] * inv;
                const u32x4 py = pack8<DT>(o);
                store16_stream(yr + col, py);
                if constexpr (DROP) {
                    // dropout of the stored (rounded) probabilities
                    float f[8];
                    unpack8<DT>(py, f);
                    const Philox rnd = dropout_bits(dk, (uint64_t)base + col);
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[j] = random16(rnd, j) < dk.threshold ? f[j] * dk.scale : 0.0f;
                    store16_stream(dropped + base + col, pack8<DT>(f));
                }
            } else if (dead[k]) {
                store16_stream(yr + col, u32x4{pd, pd, pd, pd});
                if constexpr (DROP) {
                    const float v = Half2<DT>::lo(pd);
                    float f[8];
                    const Philox rnd = dropout_bits(dk, (uint64_t)base + col);
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[j] = random16(rnd, j) < dk.threshold ? v * dk.scale : 0.0f;
                    store16_stream(dropped + base + col, pack8<DT>(f));
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Backward (causal and unmasked). dx = scale * (dy*y - y * sum(dy*y)).
// dy and y stay packed in registers between the two passes.
// ---------------------------------------------------------------------------
// EXTRA: kPlain, kPerHead (key lengths; causal only) or kDropout (dy is the gradient of
// dropout(y): the kernel first forms keep * dy / (1 - p), rounded to the storage type as the
// separate dropout backward would store it).
template <int DT, int L, int K, int W, int BW, bool CAUSAL, int EXTRA>
__global__ void __launch_bounds__((Geo<L, K, W, BW>::kThreads))
softmax_bwd_kernel(uint16_t* dx, const uint16_t* dy, const uint16_t* y, float scale,
                   uint32_t total_rows, uint32_t n, uint32_t rows_per_matrix, uint32_t window,
                   const int32_t* key_lengths, uint32_t heads, DropoutKey dk, uint32_t zshift)
{
    using G = Geo<L, K, W, BW>;
    __shared__ float lds[32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & (L - 1);
    // rotate the segment sets over the waves as in the forward kernel
    const int w = (W > 1) ? (int)((wave + (CAUSAL ? blockIdx.x : 0u)) % W) : 0;

    uint32_t row, q, mat;
    locate_row<G>(blockIdx.x, rows_per_matrix, wave, lane, L, row, q, mat);
    const bool ok = row < total_rows;
    Band band;
    if constexpr (CAUSAL) {
        band = causal_band(q, window, ok,
                           ((EXTRA & kPerHead) != 0 && ok) ? key_limit(key_lengths, mat, heads) : 0xffffffffu);
    } else {
        band.lo = 0;
        band.hi = ok ? n : 0;
    }

    const size_t base = (size_t)row * n;
    const uint32_t act = active_slots<L, K, W>(band, w);

    u32x4 rg[K], ry[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        rg[k] = u32x4{0, 0, 0, 0};
        ry[k] = u32x4{0, 0, 0, 0};
        if ((act >> k & 1u) && col < band.hi && col + 8 > band.lo) {
            rg[k] = load16_stream(dy + base + col);
            ry[k] = load16_stream(y + base + col);
            if constexpr ((EXTRA & kDropout) != 0) {
                float f[8];
                unpack8<DT>(rg[k], f);
                const Philox rnd = dropout_bits(dk, (uint64_t)base + col);
#pragma unroll
                for (int j = 0; j < 8; ++j) f[j] = random16(rnd, j) < dk.threshold ? f[j] * dk.scale : 0.0f;
                rg[k] = pack8<DT>(f);
            }
            if (CAUSAL && (col + 8 > band.hi || col < band.lo)) {
                // zero the elements outside the band (both operands): keep [a, b) of the chunk
                const uint32_t b_end = (band.hi - col < 8u) ? band.hi - col : 8u;
                const uint32_t a_beg = (band.lo > col) ? band.lo - col : 0u;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t e0 = 2u * i, e1 = 2u * i + 1u;
                    const uint32_t keep = ((e0 >= a_beg && e0 < b_end) ? 0x0000ffffu : 0u) |
                                          ((e1 >= a_beg && e1 < b_end) ? 0xffff0000u : 0u);
                    rg[k][i] &= keep;
                    ry[k][i] &= keep;
                }
            }
        }
    }

    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (act >> k & 1u) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s = fmaf(Half2<DT>::lo(rg[k][i]), Half2<DT>::lo(ry[k][i]), s);
                s = fmaf(Half2<DT>::hi(rg[k][i]), Half2<DT>::hi(ry[k][i]), s);
            }
        }
    }
    s = group_reduce<OpSum, L>(s);
    s = block_combine<OpSum, W>(s, lds, wave, lane);

    // what the formula gives where dy = y = 0 (masked columns): +0 for finite s and scale >= 0
    const float zv = scale * fmaf(-0.0f, s, 0.0f);
    const uint32_t zw = Half2<DT>::pack(zv, zv);

    // the whole row is written in one go (see the forward kernel)
    const Band wr = CAUSAL ? written_range(q, window, n, zshift) : Band{0u, n};
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = chunk_col<L, W>(k, w, l);
        if (ok && col < wr.hi && col >= wr.lo) {
            u32x4 o;
            if ((act >> k & 1u) && col < band.hi && col + 8 > band.lo) {
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

// MODE 0: causal (optional sliding window and AliBi), MODE 1: padding mask
template <int DT, int MODE>
__global__ void __launch_bounds__(kScalarThreads)
scalar_fwd_kernel(uint16_t* y, const uint16_t* x, const uint8_t* mask, float scale,
                  uint64_t n, uint64_t sq, uint64_t np, int mask_per_batch, uint32_t window,
                  const float* slopes, const uint16_t* bias, const int32_t* key_lengths, uint32_t heads,
                  uint16_t* dropped, DropoutKey dk)
{
    __shared__ float slots[4];
    const uint64_t row = blockIdx.x;
    const uint64_t q = row % sq;
    const uint16_t* xr = x + row * n;
    uint16_t* yr = y + row * n;
    const uint8_t* mrow = nullptr;
    uint64_t lo = 0, hi = n;
    float slope = 0.0f;
    const uint16_t* br = nullptr;
    uint64_t key_end = ~(uint64_t)0;  // MODE 1: keys at or beyond it count as masked
    if (MODE == 0) {
        hi = min(q + 1, (uint64_t)key_limit(key_lengths, (uint32_t)(row / sq), heads));
        lo = (q > window) ? q - window : 0;
        if (slopes != nullptr) slope = Half2<DT>::round(slopes[(row / sq) % heads]);
        if (bias != nullptr) br = bias + (((row / sq) % heads) * sq + q) * n;
    } else {
        const uint64_t bi = row / (sq * np);
        const uint64_t head = (row / sq) % np;
        mrow = mask + (mask_per_batch ? (bi * sq + q) : q) * n;
        if (slopes != nullptr) slope = Half2<DT>::round(slopes[head]);
        if (bias != nullptr) br = bias + (head * sq + q) * n;
        if (key_lengths != nullptr) key_end = key_limit(key_lengths, (uint32_t)bi, 1);
    }
    // scaled logit of column c (lo <= c < hi)
    auto logit = [&](uint64_t c) {
        float f = Half2<DT>::from_bits(xr[c]);
        if (br != nullptr) f = Half2<DT>::round(f + Half2<DT>::from_bits(br[c]));
        if (slopes != nullptr && (MODE == 0 || c <= q)) {
            const float dist = Half2<DT>::round(-(float)((int64_t)q - (int64_t)c));
            f = Half2<DT>::round(f + Half2<DT>::round(dist * slope));
        }
        float z = f * scale;
        if (MODE == 1 && (mrow[c] == 1 || c >= key_end)) z = kMaskFill;
        return z;
    };

    float m = kNegInf;
    for (uint64_t c = lo + threadIdx.x; c < hi; c += kScalarThreads) m = fmaxf(m, logit(c));
    m = block_reduce_256<OpMax>(m, slots);

    float sum = 0.0f;
    for (uint64_t c = lo + threadIdx.x; c < hi; c += kScalarThreads)
        sum += exp2_raw(fmaf(logit(c) - m, kLog2e, kExpBias));
    sum = block_reduce_256<OpSum>(sum, slots);
    const float inv = 1.0f / sum;  // an empty band (hi <= lo) never uses it

    // every thread reads and then writes the columns it owns, after the last
    // reduction barrier: y may alias x
    const bool no_key = MODE == 0 && hi <= lo;  // only key lengths can empty a causal band: a uniform row
    for (uint64_t c = threadIdx.x; c < n; c += kScalarThreads) {
        float p = no_key ? 1.0f / (float)n : 0.0f;
        if (c >= lo && c < hi) p = exp2_raw(fmaf(logit(c) - m, kLog2e, kExpBias)) * inv;
        yr[c] = Half2<DT>::to_bits(p);
        if (dropped != nullptr) {
            const uint64_t e = row * n + c;
            const Philox rnd = dropout_bits(dk, e & ~(uint64_t)7);
            const float kept = random16(rnd, (int)(e & 7u)) < dk.threshold ? Half2<DT>::round(p) * dk.scale : 0.0f;
            dropped[e] = Half2<DT>::to_bits(kept);
        }
    }
}

template <int DT, bool CAUSAL>
__global__ void __launch_bounds__(kScalarThreads)
scalar_bwd_kernel(uint16_t* dx, const uint16_t* dy, const uint16_t* y, float scale,
                  uint64_t n, uint64_t rows_per_matrix, uint32_t window, const int32_t* key_lengths, uint32_t heads,
                  int with_dropout, DropoutKey dk)
{
    __shared__ float slots[4];
    const uint64_t row = blockIdx.x;
    const uint64_t q = row % rows_per_matrix;
    const uint64_t hi =
        CAUSAL ? min(q + 1, (uint64_t)key_limit(key_lengths, (uint32_t)(row / rows_per_matrix), heads)) : n;
    const uint64_t lo = (CAUSAL && q > window) ? q - window : 0;
    const uint16_t* gr = dy + row * n;
    const uint16_t* yr = y + row * n;
    uint16_t* dr = dx + row * n;

    // the incoming gradient of column c: with dropout, keep * dy / (1 - p) rounded to the storage type
    auto grad = [&](uint64_t c) {
        float g = Half2<DT>::from_bits(gr[c]);
        if (with_dropout) {
            const uint64_t e = row * n + c;
            const Philox rnd = dropout_bits(dk, e & ~(uint64_t)7);
            g = random16(rnd, (int)(e & 7u)) < dk.threshold ? Half2<DT>::round(g * dk.scale) : 0.0f;
        }
        return g;
    };

    float s = 0.0f;
    for (uint64_t c = lo + threadIdx.x; c < hi; c += kScalarThreads) s = fmaf(grad(c), Half2<DT>::from_bits(yr[c]), s);
    s = block_reduce_256<OpSum>(s, slots);

    // each thread reads its columns of dy before it overwrites them: dx may alias dy
    for (uint64_t c = threadIdx.x; c < n; c += kScalarThreads) {
        float g = 0.0f, p = 0.0f;
        if (c >= lo && c < hi) {
            g = grad(c);
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

enum RowKind { kCausalFwd, kCausalFwdExtra, kCausalBwd, kMaskedFwd, kMaskedBwd, kMaskedFwdExtra };

// Geometry for rows of n elements, from measurements on MI355X. HBM efficiency
// drops when too many different rows are in flight per CU, and a row should be
// read and written in bursts that are compact in time, so a row is spread over
// several waves that each load about 2 KiB of it:
//   forward (one input tensor): K = 2 chunks per lane;
//   backward (two input tensors): K = 1;
//   at most 8 waves per row (workgroups of 1024 threads measured slower), so K
//   doubles for rows beyond 8 * K KiB; rows beyond 32768 elements use 16 waves;
//   padding-mask forward: as the causal forward, its waves walking over two
//   heads with one decoded mask row (measured at [16,32,1024,2048] fp16: 582 us
//   with two waves per row and two heads, 615 with four heads, 633 with one,
//   619 with one wave per row and two heads).
// The causal backward takes two chunks per lane like the forward kernels (measured by alternating shapes on the
// same tensors: 4096 keys 350 -> 346 us), and at 2048 keys three waves per row, the first of which holds two of
// the row's four segments (343 -> 335 us; block-limited 300 -> 282 us).
// blocks: the block-limited variants (a row's stores end with the block of the diagonal): four waves of four
// chunks in the forward at 8192 keys (1508 -> 1243 us with a window).
static bool plan_row(int64_t n, RowKind kind, RowPlan& p, bool blocks = false)
{
    if (n < 8 || n % 8 != 0 || n > kMaxResidentRow) return false;
    const int64_t chunks = n / 8;
    if (chunks <= 64) {
        int L = 1;
        while (L < chunks) L *= 2;
        p.L = L;
        p.K = 1;
        p.W = 1;
        return true;
    }
    p.L = 64;
    const int64_t segs = (chunks + 63) / 64;  // 1 KiB segments per row
    int W, K;
    if ((kind == kCausalFwdExtra || kind == kMaskedFwdExtra) && segs <= 4) {
        // Causal forward with per-element extra work (AliBi, bias tensor):
        // without a barrier in the row the extra instructions of one wave overlap the loads of the
        // others (measured at 2048: the extras cost 30-45 us with two waves per row, 15-20 us with one)
        W = 1;
        K = (int)segs;
    } else if (segs > 64) {
        W = 16;
        K = 8;
    } else {
        K = (kind == kCausalFwd || kind == kCausalFwdExtra || kind == kMaskedFwd || kind == kMaskedFwdExtra ||
             kind == kCausalBwd)
                ? 2
                : 1;
        while (8 * K < segs) K *= 2;
        static const int kWaves[] = {1, 2, 3, 4, 6, 8};
        W = 8;
        for (int w : kWaves)
            if ((int64_t)K * w >= segs) {
                W = w;
                break;
            }
        if ((kind == kCausalBwd || kind == kMaskedBwd) && segs == 4) {
            K = 2;  // the padding-mask backward as well: 977 -> 960 us at [16, 32, 1024, 2048]
            W = 3;
        }
        if (blocks && (kind == kCausalFwd || kind == kCausalFwdExtra) && segs > 8 && segs <= 16) {
            K = 4;
            W = 4;
        }
        // Rows of 8200..16384 keys: the kernels compiled for 8 chunks per lane (half of the slots unused here,
        // 89-100 VGPRs, 4-5 waves per SIMD) beat 4 chunks x 6 or 8 waves at full occupancy: fewer rows in
        // flight at a time (backward 67.9 -> 72.1 % of the HBM peak at 16384 keys, 69.3 -> 71.6 % at 12288;
        // forward 66.9 -> 69.6 % at 16384, but 71.3 -> 68.6 % at 12288).
        if (segs > 16 && segs <= 32 && (kind == kCausalBwd || (kind == kCausalFwd && segs > 24))) {
            K = 8;
            W = 8;
        }
    }
    p.W = NHP_TUNED_INT("NHP_W", W);
    p.K = NHP_TUNED_INT("NHP_K", K);
    if ((int64_t)p.W * p.K < segs) p.K = (int)((segs + p.W - 1) / p.W);
    return true;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The instantiated geometries (L, K, W).
#define NHP_GEOMETRIES(X)                                                                          \
    X(1, 1, 1) X(2, 1, 1) X(4, 1, 1) X(8, 1, 1) X(16, 1, 1) X(32, 1, 1) X(64, 1, 1)                \
    X(64, 2, 1) X(64, 3, 1) X(64, 4, 1)                                                            \
    X(64, 1, 2) X(64, 1, 3) X(64, 1, 4) X(64, 1, 6) X(64, 1, 8)                                    \
    X(64, 2, 2) X(64, 2, 3) X(64, 2, 4) X(64, 2, 6) X(64, 2, 8)                                    \
    X(64, 4, 4) X(64, 4, 6) X(64, 4, 8) X(64, 8, 6) X(64, 8, 8) X(64, 8, 16)

#define NHP_CASE_(L_, K_, W_) \
    case (L_) * 10000 + (K_) * 100 + (W_): CALL(L_, K_, W_); break;

// Expands CALL(L, K, W) for the plan's geometry; CALL must be defined at the point of use.
#define NHP_FOR_PLAN(PLAN)                                                 \
    do {                                                                   \
        switch ((PLAN).L * 10000 + (PLAN).K * 100 + (PLAN).W) {            \
            NHP_GEOMETRIES(NHP_CASE_)                                      \
            default: return NHP_ERR_SHAPE;                                 \
        }                                                                  \
    } while (0)

// The runtime rejects launches of 2^32 or more threads per grid dimension.
static inline bool launch_fits(int64_t blocks, int threads) { return blocks * threads < ((int64_t)1 << 32); }

constexpr int64_t kMaxRows = (int64_t)1 << 31;  // row and block ids are 32-bit on the device
constexpr uint32_t kNoWindow = 0xffffffffu;

template <int DT>
static int causal_fwd(void* y, const void* x, float scale, int64_t batches, int64_t n, uint32_t window,
                      const float* slopes, const void* bias, const int32_t* kl, uint32_t heads, hipStream_t st,
                      void* dropped = nullptr, const DropoutKey* drop = nullptr, uint32_t zshift = 0)
{
    launch_prepare();
    const int64_t rows = batches * n;
    RowPlan p;
    uint16_t* yp = static_cast<uint16_t*>(y);
    uint16_t* dp = static_cast<uint16_t*>(dropped);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* bp = static_cast<const uint16_t*>(bias);
    const DropoutKey dk = drop != nullptr ? *drop : DropoutKey{};
    const bool extras = slopes != nullptr || bp != nullptr;  // not dropout: its second output wants the two-wave shape
    const bool planned = plan_row(n, extras ? kCausalFwdExtra : kCausalFwd, p, zshift != 0) && aligned16(x) &&
                         aligned16(y) && aligned16(bias) && aligned16(dropped);
    // short rows, nothing but the mask, and enough rows for a thousand workgroups of 4 waves x R rows
    if (planned && p.K == 1 && p.W == 1 && !extras && kl == nullptr && dp == nullptr && zshift == 0 &&
        rows * p.L >= (int64_t)1024 * 256 * kShortRows) {
        const int64_t rows_per_block = (int64_t)4 * (kWave / p.L) * kShortRows;
        const uint32_t blocks = (uint32_t)((rows + rows_per_block - 1) / rows_per_block);
        if (!launch_fits(blocks, 256)) return NHP_ERR_SHAPE;
#define SHORT(L_)                                                                                      \
    case L_:                                                                                           \
        causal_fwd_short_kernel<DT, L_, kShortRows><<<blocks, 256, 0, st>>>(yp, xp, scale, (uint32_t)rows, \
                                                                           (uint32_t)n, window);       \
        break;
        switch (p.L) {
            SHORT(1) SHORT(2) SHORT(4) SHORT(8) SHORT(16) SHORT(32) SHORT(64)
        default:
            return NHP_ERR_SHAPE;
        }
#undef SHORT
        return launch_result();
    }
    if (planned) {
#define CALL(L_, K_, W_)                                                                   \
    {                                                                                      \
        using G = Geo<L_, K_, W_, kBlockWaves>;                                            \
        const uint32_t blocks = (uint32_t)((rows + G::kRowsPerBlock - 1) / G::kRowsPerBlock); \
        if (!launch_fits(blocks, G::kThreads)) return NHP_ERR_SHAPE;                       \
        const bool per_head = slopes != nullptr || bp != nullptr || kl != nullptr;         \
        /* a bias shared by several batch entries: their workgroups are interleaved (whole groups only) */ \
        uint32_t sgroup = (uint32_t)NHP_TUNED_INT("NHP_BIAS_GROUP", kBiasShareGroup);        \
        if (sgroup == 0) sgroup = (uint32_t)(n / G::kRowsPerBlock);                        \
        uint32_t sbatch = 0;                                                               \
        if (bp != nullptr && heads > 0 && batches / heads > 1 && sgroup > 0 && n % G::kRowsPerBlock == 0 && \
            (n / G::kRowsPerBlock) % sgroup == 0 && NHP_TUNED_INT("NHP_BIAS_SHARE", 1) != 0)   \
            sbatch = (uint32_t)(batches / heads);                                          \
        if (dp != nullptr && per_head)                                                     \
            causal_fwd_kernel<DT, L_, K_, W_, kBlockWaves, kPerHeadDropout><<<blocks, G::kThreads, 0, st>>>( \
                yp, xp, scale, (uint32_t)rows, (uint32_t)n, window, slopes, bp, kl, heads, dp, dk, zshift, sbatch, sgroup); \
        else if (dp != nullptr)                                                            \
            causal_fwd_kernel<DT, L_, K_, W_, kBlockWaves, kDropout><<<blocks, G::kThreads, 0, st>>>( \
                yp, xp, scale, (uint32_t)rows, (uint32_t)n, window, nullptr, nullptr, nullptr, 1, dp, dk, zshift, 0, 0); \
        else if (per_head)                                                                 \
            causal_fwd_kernel<DT, L_, K_, W_, kBlockWaves, kPerHead><<<blocks, G::kThreads, 0, st>>>( \
                yp, xp, scale, (uint32_t)rows, (uint32_t)n, window, slopes, bp, kl, heads, nullptr, dk, zshift, sbatch, sgroup); \
        else                                                                               \
            causal_fwd_kernel<DT, L_, K_, W_, kBlockWaves, kPlain><<<blocks, G::kThreads, 0, st>>>( \
                yp, xp, scale, (uint32_t)rows, (uint32_t)n, window, nullptr, nullptr, nullptr, 1, nullptr, dk, zshift, 0, 0); \
    }
        NHP_FOR_PLAN(p);
#undef CALL
    } else {
        if (!launch_fits(rows, kScalarThreads)) return NHP_ERR_SHAPE;
        scalar_fwd_kernel<DT, 0><<<(uint32_t)rows, kScalarThreads, 0, st>>>(
            yp, xp, nullptr, scale, (uint64_t)n, (uint64_t)n, 1, 0, window, slopes, bp, kl, heads, dp, dk);
    }
    return launch_result();
}

template <int DT, bool CAUSAL>
static int softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows, int64_t n,
                       int64_t rows_per_matrix, uint32_t window, const int32_t* kl, uint32_t heads, hipStream_t st,
                       const DropoutKey* drop = nullptr, uint32_t zshift = 0)
{
    launch_prepare();
    RowPlan p;
    const DropoutKey dk = drop != nullptr ? *drop : DropoutKey{};
    const bool dropout = drop != nullptr;
    uint16_t* dxp = static_cast<uint16_t*>(dx);
    const uint16_t* dyp = static_cast<const uint16_t*>(dy);
    const uint16_t* yp = static_cast<const uint16_t*>(y);
    if (plan_row(n, CAUSAL ? kCausalBwd : kMaskedBwd, p, zshift != 0) && aligned16(dx) && aligned16(dy) && aligned16(y)) {
#define CALL(L_, K_, W_)                                                                   \
    {                                                                                      \
        using G = Geo<L_, K_, W_, kBlockWaves>;                                            \
        const uint32_t blocks = (uint32_t)((rows + G::kRowsPerBlock - 1) / G::kRowsPerBlock); \
        if (!launch_fits(blocks, G::kThreads)) return NHP_ERR_SHAPE;                       \
        if (dropout && CAUSAL && kl != nullptr)                                            \
            softmax_bwd_kernel<DT, L_, K_, W_, kBlockWaves, CAUSAL, CAUSAL ? kPerHeadDropout : kDropout> \
                <<<blocks, G::kThreads, 0, st>>>(dxp, dyp, yp, scale, (uint32_t)rows, (uint32_t)n, \
                                                 (uint32_t)rows_per_matrix, window, kl, heads, dk, zshift); \
        else if (dropout)                                                                  \
            softmax_bwd_kernel<DT, L_, K_, W_, kBlockWaves, CAUSAL, kDropout>                      \
                <<<blocks, G::kThreads, 0, st>>>(dxp, dyp, yp, scale, (uint32_t)rows, (uint32_t)n, \
                                                     (uint32_t)rows_per_matrix, window, nullptr, 1, dk, zshift); \
        else if (CAUSAL && kl != nullptr)                                                  \
            softmax_bwd_kernel<DT, L_, K_, W_, kBlockWaves, CAUSAL, CAUSAL ? kPerHead : kPlain>    \
                <<<blocks, G::kThreads, 0, st>>>(dxp, dyp, yp, scale, (uint32_t)rows, (uint32_t)n, \
                                                     (uint32_t)rows_per_matrix, window, kl, heads, dk, zshift); \
        else                                                                               \
            softmax_bwd_kernel<DT, L_, K_, W_, kBlockWaves, CAUSAL, kPlain><<<blocks, G::kThreads, 0, st>>>( \
                dxp, dyp, yp, scale, (uint32_t)rows, (uint32_t)n, (uint32_t)rows_per_matrix, window, nullptr, 1, dk, \
                zshift);                                                                   \
    }
        NHP_FOR_PLAN(p);
#undef CALL
    } else {
        if (!launch_fits(rows, kScalarThreads)) return NHP_ERR_SHAPE;
        scalar_bwd_kernel<DT, CAUSAL><<<(uint32_t)rows, kScalarThreads, 0, st>>>(
            dxp, dyp, yp, scale, (uint64_t)n, (uint64_t)rows_per_matrix, window, CAUSAL ? kl : nullptr, heads,
            dropout ? 1 : 0, dk);
    }
    return launch_result();
}

// Heads a wave walks over with one decoded mask row. Two amortise the decoding;
// more make the access order less sequential and measured slower.
static uint32_t pick_heads_per_wave(int64_t np) { return (uint32_t)(np < 2 ? np : 2); }

// The extras of the padding-mask forward (all optional).
struct MaskedExtras {
    const float* slopes = nullptr;       // [np] AliBi slopes (needs sq == sk)
    const void* bias = nullptr;          // [np, sq, sk] in the scores' dtype
    const int32_t* key_lengths = nullptr;  // [b]
    bool any() const { return slopes != nullptr || bias != nullptr || key_lengths != nullptr; }
};

template <int DT>
static int masked_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b, int64_t np,
                      int64_t sq, int64_t n, int64_t pad_batches, hipStream_t st, void* dropped = nullptr,
                      const DropoutKey* drop = nullptr, const MaskedExtras& ex = MaskedExtras{})
{
    launch_prepare();
    uint16_t* dp = static_cast<uint16_t*>(dropped);
    const DropoutKey dk = drop != nullptr ? *drop : DropoutKey{};
    const int64_t bq_rows = b * sq;
    const int per_batch = (pad_batches != 1) ? 1 : 0;
    RowPlan p;
    uint16_t* yp = static_cast<uint16_t*>(y);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* bp = static_cast<const uint16_t*>(ex.bias);
    const bool mask_ok = (reinterpret_cast<uintptr_t>(mask) & 7u) == 0;
    // AliBi and the bias tensor are per-element work: one wave per row, as in the causal kernel
    const RowKind kind = (ex.slopes != nullptr || ex.bias != nullptr) ? kMaskedFwdExtra : kMaskedFwd;
    if (plan_row(n, kind, p) && aligned16(x) && aligned16(y) && aligned16(dropped) && aligned16(ex.bias) && mask_ok) {
#define LAUNCH_MASKED(L_, K_, W_, DROP_, PH_)                                                         \
    masked_fwd_kernel<DT, L_, K_, W_, kBlockWaves, DROP_, PH_><<<(uint32_t)(rb * hgs), Geo<L_, K_, W_, kBlockWaves>::kThreads, 0, st>>>( \
        yp, xp, mask, scale, (uint32_t)bq_rows, (uint32_t)sq, (uint32_t)np, (uint32_t)n, hpw, hgs, per_batch, \
        (uint32_t)rb, (uint32_t)tile, DROP_ ? dp : nullptr, dk, ex.slopes, bp, ex.key_lengths, sbatch, sgroup)
#define CALL(L_, K_, W_)                                                                   \
    {                                                                                      \
        using G = Geo<L_, K_, W_, kBlockWaves>;                                            \
        const int64_t rb = (bq_rows + G::kRowsPerBlock - 1) / G::kRowsPerBlock;            \
        const uint32_t hpw = (uint32_t)NHP_TUNED_INT("NHP_HPW", (int)pick_heads_per_wave(np)); \
        const uint32_t hgs = (uint32_t)((np + hpw - 1) / hpw);                             \
        if (rb * hgs >= kMaxRows || !launch_fits(rb * hgs, G::kThreads)) return NHP_ERR_SHAPE; \
        int64_t tile = NHP_TUNED_INT("NHP_MASK_TILE", (int)((sq + G::kRowsPerBlock - 1) / G::kRowsPerBlock)); \
        if (tile < 1) tile = 1;                                                            \
        if (tile > rb) tile = rb;                                                          \
        /* a bias shared by several batch entries: their workgroups are interleaved (tile = one batch entry) */ \
        uint32_t sgroup = (uint32_t)NHP_TUNED_INT("NHP_BIAS_GROUP", kBiasShareGroup);        \
        if (sgroup == 0) sgroup = (uint32_t)tile;                                          \
        uint32_t sbatch = 0;                                                               \
        if (bp != nullptr && b > 1 && sgroup > 0 && sq % G::kRowsPerBlock == 0 && tile == sq / G::kRowsPerBlock && \
            tile % sgroup == 0 && NHP_TUNED_INT("NHP_BIAS_SHARE", 1) != 0)                  \
            sbatch = (uint32_t)b;                                                          \
        if (dp != nullptr && ex.any())                                                     \
            LAUNCH_MASKED(L_, K_, W_, true, true);                                                     \
        else if (dp != nullptr)                                                            \
            LAUNCH_MASKED(L_, K_, W_, true, false);                                                    \
        else if (ex.any())                                                                 \
            LAUNCH_MASKED(L_, K_, W_, false, true);                                                    \
        else                                                                               \
            LAUNCH_MASKED(L_, K_, W_, false, false);                                                   \
    }
        NHP_FOR_PLAN(p);
#undef CALL
#undef LAUNCH_MASKED
    } else {
        if (!launch_fits(b * np * sq, kScalarThreads)) return NHP_ERR_SHAPE;
        scalar_fwd_kernel<DT, 1><<<(uint32_t)(b * np * sq), kScalarThreads, 0, st>>>(
            yp, xp, mask, scale, (uint64_t)n, (uint64_t)sq, (uint64_t)np, per_batch, kNoWindow, ex.slopes, bp,
            ex.key_lengths, 1, dp, dk);
    }
    return launch_result();
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int64_t nhp_softmax_max_resident_row(void) { return kMaxResidentRow; }

int nhp_softmax_geometry(int64_t row_len, int kind, int* lanes, int* chunks, int* waves)
{
    static const RowKind kKinds[] = {kCausalFwd, kCausalFwdExtra, kCausalBwd, kMaskedFwd, kMaskedBwd};
    RowPlan p;
    if (kind < 0 || kind > 4 || !plan_row(row_len, kKinds[kind], p)) return NHP_ERR_SHAPE;
    if (lanes) *lanes = p.L;
    if (chunks) *chunks = p.K;
    if (waves) *waves = p.W;
    return NHP_OK;
}

// log2 of a block size given as 0 (no blocks: 0) or a power of two >= 8; -1 for anything else
static int block_shift(int64_t zero_block)
{
    if (zero_block == 0) return 0;
    if (zero_block < 8 || zero_block > ((int64_t)1 << 30) || (zero_block & (zero_block - 1)) != 0) return -1;
    int shift = 0;
    while (((int64_t)1 << shift) < zero_block) ++shift;
    return shift;
}

int nhp_causal_softmax_blocks_fwd(void* y, const void* x, float scale, int64_t attn_batches, int64_t seq_len,
                                  int64_t window, int64_t zero_block, const float* alibi_slopes, const void* bias,
                                  const int32_t* key_lengths, int64_t heads, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    const int zshift = block_shift(zero_block);
    if (attn_batches < 0 || seq_len < 0 || zshift < 0) return NHP_ERR_SHAPE;
    const bool per_head = alibi_slopes != nullptr || bias != nullptr || key_lengths != nullptr;
    if (per_head && (heads < 1 || attn_batches % heads != 0)) return NHP_ERR_SHAPE;
    if (bias != nullptr && (bias == y)) return NHP_ERR_ALIAS;
    if (attn_batches == 0 || seq_len == 0) return NHP_OK;
    if (attn_batches > kMaxRows / seq_len - 1) return NHP_ERR_SHAPE;
    if (!x || !y) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t win = (window < 0 || window >= seq_len) ? kNoWindow : (uint32_t)window;
    const uint32_t hd = per_head ? (uint32_t)heads : 1u;
    return dtype == NHP_BF16 ? causal_fwd<NHP_BF16>(y, x, scale, attn_batches, seq_len, win, alibi_slopes, bias,
                                                    key_lengths, hd, st, nullptr, nullptr, (uint32_t)zshift)
                             : causal_fwd<NHP_F16>(y, x, scale, attn_batches, seq_len, win, alibi_slopes, bias,
                                                   key_lengths, hd, st, nullptr, nullptr, (uint32_t)zshift);
}

int nhp_causal_softmax_ex_fwd(void* y, const void* x, float scale, int64_t attn_batches, int64_t seq_len,
                              int64_t window, const float* alibi_slopes, const void* bias,
                              const int32_t* key_lengths, int64_t heads, int dtype, void* stream)
{
    return nhp_causal_softmax_blocks_fwd(y, x, scale, attn_batches, seq_len, window, 0, alibi_slopes, bias, key_lengths,
                                         heads, dtype, stream);
}

int nhp_causal_softmax_fwd(void* y, const void* x, float scale, int64_t attn_batches, int64_t seq_len,
                           int dtype, void* stream)
{
    return nhp_causal_softmax_ex_fwd(y, x, scale, attn_batches, seq_len, -1, nullptr, nullptr, nullptr, 1, dtype,
                                     stream);
}

int nhp_causal_softmax_blocks_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                                  int64_t seq_len, int64_t window, int64_t zero_block, const int32_t* key_lengths,
                                  int64_t heads, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    const int zshift = block_shift(zero_block);
    if (attn_batches < 0 || seq_len < 0 || zshift < 0) return NHP_ERR_SHAPE;
    if (key_lengths != nullptr && (heads < 1 || attn_batches % heads != 0)) return NHP_ERR_SHAPE;
    if (attn_batches == 0 || seq_len == 0) return NHP_OK;
    if (attn_batches > kMaxRows / seq_len - 1) return NHP_ERR_SHAPE;
    if (!dx || !dy || !y) return NHP_ERR_NULL;
    if (dx == y) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t rows = attn_batches * seq_len;
    const uint32_t win = (window < 0 || window >= seq_len) ? kNoWindow : (uint32_t)window;
    const uint32_t hd = key_lengths != nullptr ? (uint32_t)heads : 1u;
    return dtype == NHP_BF16 ? softmax_bwd<NHP_BF16, true>(dx, dy, y, scale, rows, seq_len, seq_len, win, key_lengths, hd,
                                                           st, nullptr, (uint32_t)zshift)
                             : softmax_bwd<NHP_F16, true>(dx, dy, y, scale, rows, seq_len, seq_len, win, key_lengths, hd,
                                                          st, nullptr, (uint32_t)zshift);
}

int nhp_causal_softmax_ex_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                              int64_t seq_len, int64_t window, const int32_t* key_lengths, int64_t heads,
                              int dtype, void* stream)
{
    return nhp_causal_softmax_blocks_bwd(dx, dy, y, scale, attn_batches, seq_len, window, 0, key_lengths, heads, dtype,
                                         stream);
}

int nhp_causal_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                           int64_t seq_len, int dtype, void* stream)
{
    return nhp_causal_softmax_ex_bwd(dx, dy, y, scale, attn_batches, seq_len, -1, nullptr, 1, dtype, stream);
}

int nhp_causal_softmax_ex_dropout_fwd(void* dropped, void* y, const void* x, float scale, int64_t attn_batches,
                                      int64_t seq_len, int64_t window, int64_t zero_block, const float* alibi_slopes,
                                      const void* bias, const int32_t* key_lengths, int64_t heads, float p,
                                      uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    const int zshift = block_shift(zero_block);
    if (attn_batches < 0 || seq_len < 0 || !(p >= 0.0f && p < 1.0f) || zshift < 0) return NHP_ERR_SHAPE;
    const bool per_head = alibi_slopes != nullptr || bias != nullptr || key_lengths != nullptr;
    if (per_head && (heads < 1 || attn_batches % heads != 0)) return NHP_ERR_SHAPE;
    if (bias != nullptr && (bias == y || bias == dropped)) return NHP_ERR_ALIAS;
    if (attn_batches == 0 || seq_len == 0) return NHP_OK;
    if (attn_batches > kMaxRows / seq_len - 1) return NHP_ERR_SHAPE;
    if (!x || !y || !dropped) return NHP_ERR_NULL;
    if (dropped == y || dropped == x) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t win = (window < 0 || window >= seq_len) ? kNoWindow : (uint32_t)window;
    const uint32_t hd = per_head ? (uint32_t)heads : 1u;
    const DropoutKey dk = make_dropout_key(p, seed, offset);
    return dtype == NHP_BF16 ? causal_fwd<NHP_BF16>(y, x, scale, attn_batches, seq_len, win, alibi_slopes, bias, key_lengths,
                                                    hd, st, dropped, &dk, (uint32_t)zshift)
                             : causal_fwd<NHP_F16>(y, x, scale, attn_batches, seq_len, win, alibi_slopes, bias, key_lengths,
                                                   hd, st, dropped, &dk, (uint32_t)zshift);
}

int nhp_causal_softmax_dropout_blocks_fwd(void* dropped, void* y, const void* x, float scale, int64_t attn_batches,
                                          int64_t seq_len, int64_t window, int64_t zero_block, float p, uint64_t seed,
                                          uint64_t offset, int dtype, void* stream)
{
    return nhp_causal_softmax_ex_dropout_fwd(dropped, y, x, scale, attn_batches, seq_len, window, zero_block, nullptr,
                                             nullptr, nullptr, 1, p, seed, offset, dtype, stream);
}

int nhp_causal_softmax_dropout_fwd(void* dropped, void* y, const void* x, float scale, int64_t attn_batches,
                                   int64_t seq_len, int64_t window, float p, uint64_t seed, uint64_t offset, int dtype,
                                   void* stream)
{
    return nhp_causal_softmax_dropout_blocks_fwd(dropped, y, x, scale, attn_batches, seq_len, window, 0, p, seed, offset,
                                                 dtype, stream);
}

int nhp_causal_softmax_ex_dropout_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                                      int64_t seq_len, int64_t window, int64_t zero_block, const int32_t* key_lengths,
                                      int64_t heads, float p, uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    const int zshift = block_shift(zero_block);
    if (attn_batches < 0 || seq_len < 0 || !(p >= 0.0f && p < 1.0f) || zshift < 0) return NHP_ERR_SHAPE;
    if (key_lengths != nullptr && (heads < 1 || attn_batches % heads != 0)) return NHP_ERR_SHAPE;
    if (attn_batches == 0 || seq_len == 0) return NHP_OK;
    if (attn_batches > kMaxRows / seq_len - 1) return NHP_ERR_SHAPE;
    if (!dx || !dy || !y) return NHP_ERR_NULL;
    if (dx == y) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t rows = attn_batches * seq_len;
    const uint32_t win = (window < 0 || window >= seq_len) ? kNoWindow : (uint32_t)window;
    const uint32_t hd = key_lengths != nullptr ? (uint32_t)heads : 1u;
    const DropoutKey dk = make_dropout_key(p, seed, offset);
    return dtype == NHP_BF16
               ? softmax_bwd<NHP_BF16, true>(dx, dy, y, scale, rows, seq_len, seq_len, win, key_lengths, hd, st, &dk, (uint32_t)zshift)
               : softmax_bwd<NHP_F16, true>(dx, dy, y, scale, rows, seq_len, seq_len, win, key_lengths, hd, st, &dk, (uint32_t)zshift);
}

int nhp_causal_softmax_dropout_blocks_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                                          int64_t seq_len, int64_t window, int64_t zero_block, float p, uint64_t seed,
                                          uint64_t offset, int dtype, void* stream)
{
    return nhp_causal_softmax_ex_dropout_bwd(dx, dy, y, scale, attn_batches, seq_len, window, zero_block, nullptr, 1, p,
                                             seed, offset, dtype, stream);
}

int nhp_causal_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, int64_t attn_batches,
                                   int64_t seq_len, int64_t window, float p, uint64_t seed, uint64_t offset, int dtype,
                                   void* stream)
{
    return nhp_causal_softmax_dropout_blocks_bwd(dx, dy, y, scale, attn_batches, seq_len, window, 0, p, seed, offset, dtype,
                                                 stream);
}

// Shared argument checks of the padding-mask forward entry points.
static int masked_fwd_check(const void* y, const void* x, const uint8_t* mask, int64_t b, int64_t np, int64_t sq,
                            int64_t sk, int64_t pad_batches, const MaskedExtras& ex, int dtype, bool& empty)
{
    empty = false;
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    if (b < 0 || np < 0 || sq < 0 || sk < 0) return NHP_ERR_SHAPE;
    if (ex.slopes != nullptr && sq != sk) return NHP_ERR_SHAPE;  // the AliBi bias is defined on square scores
    if (b == 0 || np == 0 || sq == 0 || sk == 0) {
        empty = true;
        return NHP_OK;
    }
    if (pad_batches != 1 && pad_batches != b) return NHP_ERR_PAD_BATCHES;
    if (b > kMaxRows / np - 1 || b * np > kMaxRows / sq - 1) return NHP_ERR_SHAPE;
    if (!x || !y || !mask) return NHP_ERR_NULL;
    if (ex.bias != nullptr && ex.bias == y) return NHP_ERR_ALIAS;
    return NHP_OK;
}

int nhp_masked_softmax_ex_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b, int64_t np,
                              int64_t sq, int64_t sk, int64_t pad_batches, const float* alibi_slopes, const void* bias,
                              const int32_t* key_lengths, int dtype, void* stream)
{
    MaskedExtras ex;
    ex.slopes = alibi_slopes;
    ex.bias = bias;
    ex.key_lengths = key_lengths;
    bool empty;
    const int rc = masked_fwd_check(y, x, mask, b, np, sq, sk, pad_batches, ex, dtype, empty);
    if (rc != NHP_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dtype == NHP_BF16 ? masked_fwd<NHP_BF16>(y, x, mask, scale, b, np, sq, sk, pad_batches, st, nullptr, nullptr, ex)
                             : masked_fwd<NHP_F16>(y, x, mask, scale, b, np, sq, sk, pad_batches, st, nullptr, nullptr, ex);
}

int nhp_masked_softmax_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b,
                           int64_t np, int64_t sq, int64_t sk, int64_t pad_batches, int dtype,
                           void* stream)
{
    return nhp_masked_softmax_ex_fwd(y, x, mask, scale, b, np, sq, sk, pad_batches, nullptr, nullptr, nullptr, dtype,
                                     stream);
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
    return dtype == NHP_BF16 ? softmax_bwd<NHP_BF16, false>(dx, dy, y, scale, rows, sk, rows, kNoWindow, nullptr, 1, st)
                             : softmax_bwd<NHP_F16, false>(dx, dy, y, scale, rows, sk, rows, kNoWindow, nullptr, 1, st);
}

int nhp_masked_softmax_ex_dropout_fwd(void* dropped, void* y, const void* x, const uint8_t* mask, float scale,
                                      int64_t b, int64_t np, int64_t sq, int64_t sk, int64_t pad_batches,
                                      const float* alibi_slopes, const void* bias, const int32_t* key_lengths, float p,
                                      uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    MaskedExtras ex;
    ex.slopes = alibi_slopes;
    ex.bias = bias;
    ex.key_lengths = key_lengths;
    bool empty;
    if (!(p >= 0.0f && p < 1.0f)) return (dtype != NHP_F16 && dtype != NHP_BF16) ? NHP_ERR_DTYPE : NHP_ERR_SHAPE;
    const int rc = masked_fwd_check(y, x, mask, b, np, sq, sk, pad_batches, ex, dtype, empty);
    if (rc != NHP_OK || empty) return rc;
    if (!dropped) return NHP_ERR_NULL;
    if (dropped == y || dropped == x || (bias != nullptr && dropped == bias)) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const DropoutKey dk = make_dropout_key(p, seed, offset);
    return dtype == NHP_BF16 ? masked_fwd<NHP_BF16>(y, x, mask, scale, b, np, sq, sk, pad_batches, st, dropped, &dk, ex)
                             : masked_fwd<NHP_F16>(y, x, mask, scale, b, np, sq, sk, pad_batches, st, dropped, &dk, ex);
}

int nhp_masked_softmax_dropout_fwd(void* dropped, void* y, const void* x, const uint8_t* mask, float scale,
                                   int64_t b, int64_t np, int64_t sq, int64_t sk, int64_t pad_batches, float p,
                                   uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    return nhp_masked_softmax_ex_dropout_fwd(dropped, y, x, mask, scale, b, np, sq, sk, pad_batches, nullptr, nullptr,
                                             nullptr, p, seed, offset, dtype, stream);
}

int nhp_masked_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows, int64_t sk,
                                   float p, uint64_t seed, uint64_t offset, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16) return NHP_ERR_DTYPE;
    if (rows < 0 || sk < 0 || !(p >= 0.0f && p < 1.0f)) return NHP_ERR_SHAPE;
    if (rows == 0 || sk == 0) return NHP_OK;
    if (rows >= kMaxRows) return NHP_ERR_SHAPE;
    if (!dx || !dy || !y) return NHP_ERR_NULL;
    if (dx == y) return NHP_ERR_ALIAS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const DropoutKey dk = make_dropout_key(p, seed, offset);
    return dtype == NHP_BF16
               ? softmax_bwd<NHP_BF16, false>(dx, dy, y, scale, rows, sk, rows, kNoWindow, nullptr, 1, st, &dk)
               : softmax_bwd<NHP_F16, false>(dx, dy, y, scale, rows, sk, rows, kNoWindow, nullptr, 1, st, &dk);
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
