// Fused rotary positional embedding (rotate-half form), forward and backward,
// for gfx950.
//
// Tensor t is [s, b, h, d] with arbitrary element strides; the first d2
// elements of every head vector are rotated with the angle of position s,
// the remaining d - d2 are copied.
//
// Vector kernels. A head vector is cut into 16-byte chunks (V = 8 elements for
// 16-bit data, 4 for fp32) and every lane owns one chunk, so a wave-wide load
// or store moves up to 1 KiB of consecutive head vectors. The rotation pairs
// element i with i + d2/2, i.e. a chunk with the chunk d2/(2V) lanes away in
// the same wave; the partner's data is fetched with ds_bpermute (no memory
// traffic). Chunks of the pass-through tail are copied by their lanes.
//   rope_lean_kernel: two chunks per thread, no loop, every load issued before
//     the first wait: the shape a plain streaming copy runs fastest in on this
//     GPU. Head vectors of any number of chunks up to 64.
//   rope_vec_kernel: what the lean kernel's grid cannot hold (more than 65535
//     positions) and calls without a rotary part. A workgroup stays on one sequence
//     position and walks over the (batch, head) rows, re-using the cos/sin values it loaded once.
//   When the angles are given instead of cached tables, a workgroup of either
//   kernel first evaluates sin and cos of its position, one rotary feature per
//   thread, into LDS (sincosf costs a few hundred instructions: evaluated per
//   lane it made these kernels compute-bound).
//
//   Rotary dimensions whose half is not a whole number of chunks (24 of 96,
//     20 of 80) or unaligned tables: partner elements are picked from LDS one by
//     one, by a variant of the lean kernel (rope_gather_kernel beyond its grid).
//
// Transposing kernel, for 16-bit inputs that are contiguous along the sequence
// instead of along the features (see rope_tr_kernel). Everything else (odd
// sizes, unaligned pointers, other strides) takes the scalar kernel.
//
// Arithmetic: out = (x (*) c) (+) (r (*) s) where every product and the sum
// are rounded to the data dtype, which is what the scalar types of the
// reference kernels and eager torch do.

#include "common.hpp"

namespace nhp {

// out = round(round(x*c) +/- round(r*s)); the three roundings of the scalar types.
// Negating r or s before the product equals subtracting the rounded product
// (rounding to nearest is symmetric), so the sign is taken as a flag.
template <int DT, bool NEG = false>
__device__ __forceinline__ float rot(float x, float c, float r, float s)
{
    const float p1 = Elt<DT>::round(x * c);
    const float p2 = Elt<DT>::round(r * s);
    return Elt<DT>::round(NEG ? p1 - p2 : p1 + p2);
}

// ---------------------------------------------------------------------------
// Sources of cos/sin. `get(pos, i, c, s)` returns cos and sin of element i of
// position pos, already rounded to the data dtype.
// ---------------------------------------------------------------------------
template <int DT, int CS>  // CS: dtype of the cached tables
struct CachedTables {
    static constexpr bool kEvaluate = false;
    const void* cos;
    const void* sin;
    int64_t d2;
    __device__ __forceinline__ void get(int64_t pos, int64_t i, float& c, float& s) const
    {
        c = Elt<DT>::round(Elt<CS>::load(cos, pos * d2 + i));
        s = Elt<DT>::round(Elt<CS>::load(sin, pos * d2 + i));
    }
    // V consecutive values starting at element i (i % V == 0, tables 16-byte aligned)
    __device__ __forceinline__ void get_vec(int64_t pos, int64_t i, float (&c)[Elt<DT>::kVec],
                                            float (&s)[Elt<DT>::kVec]) const
    {
        constexpr int V = Elt<DT>::kVec;
        if constexpr (CS == DT) {
            chunk_to_float<DT>(load16(static_cast<const typename Elt<CS>::storage*>(cos) + pos * d2 + i), c);
            chunk_to_float<DT>(load16(static_cast<const typename Elt<CS>::storage*>(sin) + pos * d2 + i), s);
        } else {
            // fp32 tables with 16-bit data: two 16-byte loads per table
            const float* cp = static_cast<const float*>(cos) + pos * d2 + i;
            const float* sp = static_cast<const float*>(sin) + pos * d2 + i;
#pragma unroll
            for (int v = 0; v < V; v += 4) {
                const u32x4 a = load16(cp + v);
                const u32x4 b = load16(sp + v);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    c[v + t] = Elt<DT>::round(bitcast<float>(a[t]));
                    s[v + t] = Elt<DT>::round(bitcast<float>(b[t]));
                }
            }
        }
    }
};

template <int DT>
struct FreqTable {
    // sin and cos are evaluated on the device: the vector kernels do it once per workgroup and
    // position, into LDS, instead of once per lane
    static constexpr bool kEvaluate = true;
    const float* freqs;
    int64_t d2;
    __device__ __forceinline__ void get(int64_t pos, int64_t i, float& c, float& s) const
    {
        float sv, cv;
        sincosf(freqs[pos * d2 + i], &sv, &cv);
        c = Elt<DT>::round(cv);
        s = Elt<DT>::round(sv);
    }
    __device__ __forceinline__ void get_vec(int64_t pos, int64_t i, float (&c)[Elt<DT>::kVec],
                                            float (&s)[Elt<DT>::kVec]) const
    {
#pragma unroll
        for (int v = 0; v < Elt<DT>::kVec; ++v) get(pos, i + v, c[v], s[v]);
    }
};

// Rotary features a vector kernel can take: d <= 64 chunks of at most 8 elements.
constexpr int kMaxRotary = 512;

// cos/sin of position `pos` for the workgroup: with evaluated tables the first d2 threads compute one
// value each into LDS (every thread of the workgroup has to call this: it holds a barrier).
template <typename Tables>
__device__ __forceinline__ void stage_tables(const Tables& tab, int64_t pos, int d2, float* tcos, float* tsin)
{
    if constexpr (Tables::kEvaluate) {
        for (int i = (int)threadIdx.x; i < d2; i += (int)blockDim.x) tab.get(pos, i, tcos[i], tsin[i]);
        __syncthreads();
    }
}

// V consecutive values of the staged tables, or of the cached ones.
template <int DT, typename Tables>
__device__ __forceinline__ void table_chunk(const Tables& tab, int64_t pos, int e, const float* tcos, const float* tsin,
                                            float (&c)[Elt<DT>::kVec], float (&s)[Elt<DT>::kVec])
{
    if constexpr (Tables::kEvaluate) {
#pragma unroll
        for (int v = 0; v < Elt<DT>::kVec; ++v) {
            c[v] = tcos[e + v];
            s[v] = tsin[e + v];
        }
    } else {
        tab.get_vec(pos, (int64_t)e, c, s);
    }
}

// ---------------------------------------------------------------------------
// Vector kernel
//   grid  = (s, row_splits), block = 256 threads = 4 waves
//   lane  = (row within wave) * cpr + chunk,  cpr = d / V chunks per head vector
//   a wave covers rpw = 64 / cpr rows per step, the workgroup 4 * rpw, and the
//   workgroups of one position interleave over the b*h rows.
// Requires: stride_d == 1 on both sides, d % V == 0, d2 % (2V) == 0, d <= 64 V,
// every other stride a multiple of V, 16-byte aligned base pointers and tables.
// ---------------------------------------------------------------------------
// One tensor of a launch: where it lives and how its (batch, head) rows are strided.
struct RopeTensor {
    void* out;
    const void* in;
    int rows;  // b * h
    int h;
    int64_t is_s, is_b, is_h, os_s, os_b, os_h;
};
// A launch rotates one or two tensors (q and k) with the same tables; blockIdx.z picks the tensor.
struct RopePair {
    RopeTensor t[2];
};

// FLAT: the batch and head dimensions collapse into one row dimension on both
// sides (stride_b == h * stride_h), which saves the division by h per row.
// U: rows in flight per lane (loads of U steps are issued before the first is used).
template <int DT, bool BWD, bool FLAT, int U, typename Tables>
__global__ void __launch_bounds__(256)
rope_vec_kernel(RopePair pair, Tables tab, int cpr, int rot_chunks, int rpw)
{
    const RopeTensor& T = pair.t[blockIdx.z];
    void* const out = T.out;
    const void* const in = T.in;
    const int rows = T.rows, h = T.h;
    const int64_t is_s = T.is_s, is_b = T.is_b, is_h = T.is_h, os_s = T.os_s, os_b = T.os_b, os_h = T.os_h;
    constexpr int V = Elt<DT>::kVec;
    using S = typename Elt<DT>::storage;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int rl = lane / cpr;        // row within the wave's group
    const int c = lane - rl * cpr;    // chunk within the head vector
    const bool lane_on = rl < rpw;
    const int64_t pos = blockIdx.x;
    __shared__ float tcos[Tables::kEvaluate ? kMaxRotary : 1], tsin[Tables::kEvaluate ? kMaxRotary : 1];
    stage_tables(tab, pos, rot_chunks * V, tcos, tsin);

    const int half = rot_chunks / 2;
    const bool is_rot = c < rot_chunks;
    const bool first = c < half;
    const int partner_lane = is_rot ? (first ? lane + half : lane - half) : lane;

    // cos of the own chunk; sin of the own chunk (forward) or of the partner's (backward)
    float cv[V], sv[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        cv[v] = 0.0f;
        sv[v] = 0.0f;
    }
    if (lane_on && is_rot) {
        float unused[V];
        if (!BWD) {
            table_chunk<DT>(tab, pos, c * V, tcos, tsin, cv, sv);
        } else {
            table_chunk<DT>(tab, pos, c * V, tcos, tsin, cv, unused);
            table_chunk<DT>(tab, pos, (first ? c + half : c - half) * V, tcos, tsin, unused, sv);
        }
    }
    // forward: first half subtracts, backward: second half subtracts
    const bool negate = BWD ? !first : first;

    const S* ip = static_cast<const S*>(in) + pos * is_s + (int64_t)c * V;
    S* op = static_cast<S*>(out) + pos * os_s + (int64_t)c * V;

    const int rows_per_step = 4 * rpw;
    const int stride = rows_per_step * (int)gridDim.y;
    // All lanes of a row (a lane and its partner included) share r0 and leave the loop together.
    for (int r0 = (int)blockIdx.y * rows_per_step + wave * rpw + rl; r0 < rows; r0 += stride * U) {
        u32x4 raw[U];
        int64_t dst_off[U];
        bool on[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = r0 + u * stride;
            on[u] = lane_on && r < rows;
            raw[u] = u32x4{0, 0, 0, 0};
            dst_off[u] = 0;
            if (on[u]) {
                if (FLAT) {
                    raw[u] = load16_stream(ip + r * is_h);
                    dst_off[u] = r * os_h;
                } else {
                    const int bi = r / h;
                    const int hi = r - bi * h;
                    raw[u] = load16_stream(ip + bi * is_b + hi * is_h);
                    dst_off[u] = bi * os_b + hi * os_h;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            u32x4 praw;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                praw[i] = (uint32_t)__builtin_amdgcn_ds_bpermute(partner_lane << 2, (int)raw[u][i]);
            u32x4 res = raw[u];
            if (is_rot) {
                float x[V], pr[V], y[V];
                chunk_to_float<DT>(raw[u], x);
                chunk_to_float<DT>(praw, pr);
#pragma unroll
                for (int v = 0; v < V; ++v)
                    y[v] = negate ? rot<DT, true>(x[v], cv[v], pr[v], sv[v]) : rot<DT>(x[v], cv[v], pr[v], sv[v]);
                res = float_to_chunk<DT>(y);
            }
            if (on[u]) store16_stream(op + dst_off[u], res);
        }
    }
}

// ---------------------------------------------------------------------------
// Gather kernel: rotary dimensions whose half is not a whole number of chunks
// (d2 = 24 of 96, 20 of 80: a quarter of the head sizes 96 and 80), or tables
// that are not 16-byte aligned. The launch shape of rope_vec_kernel; a lane
// still owns one chunk, but the partner of element i, i +- d2/2, may sit
// anywhere in up to two other chunks of the head vector, so every lane puts
// its chunk into LDS and picks its partner elements from there one by one
// (the lanes of a head vector share a wave, whose LDS accesses execute in
// order: a wave-level fence is all the synchronisation needed). cos and sin of
// the position are staged in LDS by the workgroup whatever their source.
// Requires: stride_d == 1 on both sides, d % V == 0, d <= 64 V, d2 even, every
// other stride a multiple of V, 16-byte aligned base pointers.
// ---------------------------------------------------------------------------
template <int DT, bool BWD, bool FLAT, int U, typename Tables>
__global__ void __launch_bounds__(256)
rope_gather_kernel(RopePair pair, Tables tab, int cpr, int d2, int rpw)
{
    const RopeTensor& T = pair.t[blockIdx.z];
    void* const out = T.out;
    const void* const in = T.in;
    const int rows = T.rows, h = T.h;
    const int64_t is_s = T.is_s, is_b = T.is_b, is_h = T.is_h, os_s = T.os_s, os_b = T.os_b, os_h = T.os_h;
    constexpr int V = Elt<DT>::kVec;
    using S = typename Elt<DT>::storage;
    __shared__ float tcos[kMaxRotary], tsin[kMaxRotary];
    __shared__ u32x4 stage[U][256];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int rl = lane / cpr;
    const int c = lane - rl * cpr;
    const bool lane_on = rl < rpw;
    const int64_t pos = blockIdx.x;

    for (int i = (int)threadIdx.x; i < d2; i += 256) tab.get(pos, i, tcos[i], tsin[i]);
    __syncthreads();

    // per element of the own chunk: cos, the sine the formula takes (its own forward, the partner's
    // backward), the sign, and where the partner sits among the staged elements of the head vector
    const int h2 = d2 / 2;
    const int vec0 = ((int)threadIdx.x - c) * V;  // first staged element of this lane's head vector
    float cv[V], sv[V];
    int src[V];
    bool neg[V];
    bool any = false;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int i = c * V + v;
        const bool rot_on = lane_on && i < d2;
        const bool first = i < h2;
        const int pi = first ? i + h2 : i - h2;
        cv[v] = rot_on ? tcos[i] : 0.0f;
        sv[v] = rot_on ? tsin[BWD ? pi : i] : 0.0f;
        neg[v] = BWD ? !first : first;
        src[v] = rot_on ? vec0 + pi : -1;
        any = any || rot_on;
    }

    const S* ip = static_cast<const S*>(in) + pos * is_s + (int64_t)c * V;
    S* op = static_cast<S*>(out) + pos * os_s + (int64_t)c * V;
    const int rows_per_step = 4 * rpw;
    const int stride = rows_per_step * (int)gridDim.y;
    for (int r0 = (int)blockIdx.y * rows_per_step + wave * rpw + rl; r0 < rows; r0 += stride * U) {
        u32x4 raw[U];
        int64_t dst_off[U];
        bool on[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = r0 + u * stride;
            on[u] = lane_on && r < rows;
            raw[u] = u32x4{0, 0, 0, 0};
            dst_off[u] = 0;
            if (on[u]) {
                if (FLAT) {
                    raw[u] = load16_stream(ip + r * is_h);
                    dst_off[u] = r * os_h;
                } else {
                    const int bi = r / h;
                    const int hi = r - bi * h;
                    raw[u] = load16_stream(ip + bi * is_b + hi * is_h);
                    dst_off[u] = bi * os_b + hi * os_h;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) stage[u][threadIdx.x] = raw[u];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int u = 0; u < U; ++u) {
            u32x4 res = raw[u];
            if (any) {
                const S* staged = reinterpret_cast<const S*>(&stage[u][0]);
                float x[V], y[V];
                chunk_to_float<DT>(raw[u], x);
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    y[v] = x[v];
                    if (src[v] >= 0) {
                        float pr;
                        if constexpr (DT == NHP_F32)
                            pr = staged[src[v]];
                        else
                            pr = Half2<DT>::from_bits(staged[src[v]]);
                        y[v] = neg[v] ? rot<DT, true>(x[v], cv[v], pr, sv[v]) : rot<DT>(x[v], cv[v], pr, sv[v]);
                    }
                }
                res = float_to_chunk<DT>(y);
            }
            if (on[u]) store16_stream(op + dst_off[u], res);
        }
        // the next iteration overwrites the staged chunks: its stores follow these loads in program order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

// ---------------------------------------------------------------------------
// Lean vector kernel
//   grid  = (ceil(rows / (8 * RPW)), s, tensors), block = 256 threads = 4 waves
//   A head vector is CPR chunks; a wave holds RPW = 64 / CPR whole head vectors (its last 64 - RPW * CPR lanes
//   idle when CPR is not a power of two: 4 of 64 at 12 chunks), consecutive waves consecutive rows, and every
//   thread owns the same chunk of two rows, 4 * RPW rows apart, so that both share one pair of table chunks.
//   LOG_CPR >= 0: CPR = 2^LOG_CPR at compile time; LOG_CPR < 0: any CPR <= 64, passed as an argument.
// Consecutive workgroups sweep consecutive memory. Every load (tables, then
// data) is issued before anything waits: lanes outside the rotary part load
// table chunk 0 and discard the result, a second row beyond the end re-loads
// the last row and is not stored, so that no load sits in a divergent region
// (where the compiler would have to wait for it on the spot, or would sink it
// behind the wait for the data). Needs d2 > 0.
//
// JOINT: q and k are slices of one buffer with k's head vectors directly behind q's (k.in == q.in + d, equal
// strides, equal row counts: how the attention layer slices them from its fused projection,
// megatron/model/transformer.py:852-866). The two head vectors of a row are then read as one run of 2 * CPR
// chunks, whose first half goes to q's output and whose second half to k's: one pass over the buffer instead
// of two that each pick every third head vector. `ta` describes q (and both inputs), `tb.out` is k's output.
//
// GATHER: rotary dimensions whose half is not a whole number of chunks (24 of 96, 20 of 80: a quarter of
// the head sizes 96 and 80), or tables that are not 16-byte aligned. The partner of element i, i +- d2/2, may
// sit anywhere in up to two other chunks of the head vector, so every lane puts its chunks into LDS and
// picks its partner elements from there one by one (the lanes of a head vector share a wave, whose LDS
// accesses execute in order: a wave-level fence is all the synchronisation needed); cos and sin of the
// position are staged in LDS by the workgroup whatever their source. `rot_arg` is then d2, else d2 / V.
// ---------------------------------------------------------------------------
constexpr int kLeanThreads = 256;
constexpr int kLeanU = 2;

template <int DT, bool BWD, int LOG_CPR, bool FLAT, typename Tables, bool JOINT = false, bool GATHER = false>
__global__ void __launch_bounds__(kLeanThreads)
rope_lean_kernel(RopeTensor ta, RopeTensor tb, Tables tab, int rot_arg, int cpr_arg)
{
    static_assert(!(JOINT && (GATHER || LOG_CPR < 0)), "the joint variant exists for power-of-two head vectors only");
    constexpr int V = Elt<DT>::kVec;
    constexpr int U = kLeanU;
    constexpr bool STAGED = GATHER || Tables::kEvaluate;  // cos and sin come from LDS
    using S = typename Elt<DT>::storage;
    // both tensors' descriptions arrive with the kernel arguments; blockIdx.z picks one
    const bool second = !JOINT && blockIdx.z != 0;
    const S* const in = static_cast<const S*>(second ? tb.in : ta.in);
    S* const out = static_cast<S*>(second ? tb.out : ta.out);
    const int rows = second ? tb.rows : ta.rows;
    const int h = second ? tb.h : ta.h;
    const int64_t is_s = second ? tb.is_s : ta.is_s, is_b = second ? tb.is_b : ta.is_b, is_h = second ? tb.is_h : ta.is_h;
    const int64_t os_s = second ? tb.os_s : ta.os_s, os_b = second ? tb.os_b : ta.os_b, os_h = second ? tb.os_h : ta.os_h;

    const int cpr = LOG_CPR >= 0 ? (1 << (LOG_CPR >= 0 ? LOG_CPR : 0)) : cpr_arg;  // chunks per head vector
    const int run = JOINT ? 2 * cpr : cpr;  // chunks a row contributes: one head vector, or q's and k's
    const int rpw = 64 / run;               // rows per wave
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int rl = lane / run;              // row within the wave
    const int cj = lane - rl * run;         // chunk within the row's run
    const int c = JOINT ? (cj & (cpr - 1)) : cj;  // chunk within its head vector
    const int64_t pos = blockIdx.y;
    const int d2 = GATHER ? rot_arg : rot_arg * V;
    __shared__ float tcos[STAGED ? kMaxRotary : 1], tsin[STAGED ? kMaxRotary : 1];
    __shared__ u32x4 stage[GATHER ? U : 1][GATHER ? kLeanThreads : 1];
    if constexpr (GATHER) {
        for (int i = (int)threadIdx.x; i < d2; i += kLeanThreads) tab.get(pos, i, tcos[i], tsin[i]);
        __syncthreads();
    } else {
        stage_tables(tab, pos, d2, tcos, tsin);
    }
    const int r0 = ((int)blockIdx.x * (4 * U) + wave) * rpw + rl;
    if (rl < rpw && r0 < rows) {
        // addresses first, then all loads back to back
        const S* ip = in + pos * is_s + cj * V;
        S* op = ((JOINT && cj >= cpr) ? static_cast<S*>(tb.out) : out) + pos * os_s + c * V;
        int64_t src[U], dst[U];
        bool on[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = r0 + u * 4 * rpw;
            on[u] = r < rows;
            const int rr = on[u] ? r : rows - 1;
            if (FLAT) {
                src[u] = rr * is_h;
                dst[u] = rr * os_h;
            } else {
                const int bi = rr / h;
                const int hi = rr - bi * h;
                src[u] = bi * is_b + hi * is_h;
                dst[u] = bi * os_b + hi * os_h;
            }
        }
        if constexpr (!GATHER) {
            const int rot_chunks = rot_arg;
            const int half = rot_chunks >> 1;
            const bool is_rot = c < rot_chunks;
            const bool first = c < half;
            const int partner_lane = is_rot ? (first ? lane + half : lane - half) : lane;
            // cos of the own chunk; sin of the own chunk (forward) or of the partner's (backward)
            const int tc = is_rot ? c : 0;
            const int ts = is_rot ? (BWD ? (first ? c + half : c - half) : c) : 0;
            float cv[V], sv[V], unused[V];
            table_chunk<DT>(tab, pos, tc * V, tcos, tsin, cv, unused);
            table_chunk<DT>(tab, pos, ts * V, tcos, tsin, unused, sv);
            u32x4 raw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) raw[u] = load16_stream(ip + src[u]);
            // forward: first half subtracts, backward: second half subtracts
            const bool negate = BWD ? !first : first;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                u32x4 praw;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    praw[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(partner_lane << 2, (int)raw[u][k]);
                float x[V], pr[V], y[V];
                chunk_to_float<DT>(raw[u], x);
                chunk_to_float<DT>(praw, pr);
#pragma unroll
                for (int v = 0; v < V; ++v)
                    y[v] = negate ? rot<DT, true>(x[v], cv[v], pr[v], sv[v]) : rot<DT>(x[v], cv[v], pr[v], sv[v]);
                const u32x4 rotated = float_to_chunk<DT>(y);
                u32x4 res;
#pragma unroll
                for (int k = 0; k < 4; ++k) res[k] = is_rot ? rotated[k] : raw[u][k];
                // The value passes through an opaque statement: without it the compiler folds the select into
                // the store and the store loses its non-temporal hint.
                asm volatile("" : "+v"(res));
                if (on[u]) store16_stream(op + dst[u], res);
            }
        } else if ((d2 >> 1) % (4 / (int)sizeof(S)) == 0 && d2 % (4 / (int)sizeof(S)) == 0) {
            // Half the rotary dimension is a whole number of 32-bit words (12 of 24 elements, 10 of 20): the
            // partner of every word of the own chunk is a whole word somewhere in the head vector. Four 32-bit
            // LDS reads with addresses fixed per lane replace the chunk exchange of the plain variant; the
            // arithmetic is then the same, a whole chunk at a time. The sign of the rotated term is folded
            // into the sine (r * (-s) is -(r * s) exactly, and a + (-b) is a - b).
            constexpr int E = 4 / (int)sizeof(S);  // elements per word
            u32x4 raw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) raw[u] = load16_stream(ip + src[u]);
            const int h2 = d2 >> 1;
            const int h2w = h2 / E, d2w = d2 / E;
            const int vecw0 = ((int)threadIdx.x - c) * 4;  // first staged word of this lane's head vector
            int from[4];
            bool turns[4];
            float cv[V], sv[V];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int w = c * 4 + k;
                turns[k] = w < d2w;
                const bool first = w < h2w;
                const int pw = turns[k] ? (first ? w + h2w : w - h2w) : w;
                // lanes outside the rotary part read a word they do not use: one per lane and bank (their own
                // chunk's words, 4 words apart from lane to lane, would make every such read a 4-way bank conflict)
                from[k] = turns[k] ? vecw0 + pw : (int)threadIdx.x;
                const bool negate = BWD ? !first : first;
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const int i = w * E + e, pi = pw * E + e;
                    cv[k * E + e] = turns[k] ? tcos[i] : 0.0f;
                    const float sn = turns[k] ? tsin[BWD ? pi : i] : 0.0f;
                    sv[k * E + e] = negate ? -sn : sn;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) stage[u][threadIdx.x] = raw[u];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t* words = reinterpret_cast<const uint32_t*>(&stage[u][0]);
                u32x4 praw;
#pragma unroll
                for (int k = 0; k < 4; ++k) praw[k] = words[from[k]];
                float x[V], pr[V], y[V];
                chunk_to_float<DT>(raw[u], x);
                chunk_to_float<DT>(praw, pr);
#pragma unroll
                for (int v = 0; v < V; ++v) y[v] = rot<DT>(x[v], cv[v], pr[v], sv[v]);
                const u32x4 rotated = float_to_chunk<DT>(y);
                u32x4 res;
#pragma unroll
                for (int k = 0; k < 4; ++k) res[k] = turns[k] ? rotated[k] : raw[u][k];
                asm volatile("" : "+v"(res));
                if (on[u]) store16_stream(op + dst[u], res);
            }
        } else {
            u32x4 raw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) raw[u] = load16_stream(ip + src[u]);
            // per element of the own chunk: cos, the sine the formula takes (its own forward, the partner's
            // backward), the sign, and where the partner sits among the staged elements of the head vector
            const int h2 = d2 >> 1;
            const int vec0 = ((int)threadIdx.x - c) * V;  // first staged element of this lane's head vector
            float cv[V], sv[V];
            int from[V];
            bool neg[V];
            bool any = false;
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const int i = c * V + v;
                const bool rot_on = i < d2;
                const bool first = i < h2;
                const int pi = first ? i + h2 : i - h2;
                cv[v] = rot_on ? tcos[i] : 0.0f;
                sv[v] = rot_on ? tsin[BWD ? pi : i] : 0.0f;
                neg[v] = BWD ? !first : first;
                from[v] = rot_on ? vec0 + pi : -1;
                any = any || rot_on;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) stage[u][threadIdx.x] = raw[u];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int u = 0; u < U; ++u) {
                u32x4 res = raw[u];
                if (any) {
                    const S* staged = reinterpret_cast<const S*>(&stage[u][0]);
                    float x[V], y[V];
                    chunk_to_float<DT>(raw[u], x);
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        y[v] = x[v];
                        if (from[v] >= 0) {
                            float pr;
                            if constexpr (DT == NHP_F32)
                                pr = staged[from[v]];
                            else
                                pr = Half2<DT>::from_bits(staged[from[v]]);
                            y[v] = neg[v] ? rot<DT, true>(x[v], cv[v], pr, sv[v]) : rot<DT>(x[v], cv[v], pr, sv[v]);
                        }
                    }
                    res = float_to_chunk<DT>(y);
                }
                asm volatile("" : "+v"(res));
                if (on[u]) store16_stream(op + dst[u], res);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Transposing kernel: the input is contiguous along the sequence (stride_s == 1,
// features stride_d apart), the output along the features. This is the layout in
// which the gradient of the keys arrives from the backward of the score GEMM
// (q k^T hands its second operand's gradient over as [b, h, d, s]).
//   grid  = (b * h rows, ceil(s / 64)), block = 256 threads
//   phase 1: 16-byte loads along s. A wave covers, per pass, the 8 features of one
//            output chunk (lane >> 3) by the 64 positions of the tile (8 lanes of 8
//            positions each). The 8 x 8 block of 16-bit elements that 8 lanes 8 apart
//            hold is transposed in registers (one DPP exchange, then the row and
//            half-wave swaps of gfx950), after which every lane owns one whole output
//            chunk and writes it to LDS with one 16-byte store; the chunk slot is
//            XOR-ed with the position group so that neither side conflicts
//   phase 2: one lane per (position, feature chunk) reads its chunk and the
//            partner chunk from LDS, rotates, and stores 16 bytes. With a partial
//            rotary dimension the rotation is done first, in place in LDS, by as
//            many lanes as there are rotating chunk pairs (all of them busy), and
//            the tile is then copied out without arithmetic
// 16-bit data only; P = ceil(d / 32) load passes, all in flight together.
// Requires: s % 8 == 0, stride_d and the batch / head strides multiples of 8,
// output stride_d == 1, aligned pointers, d % 8 == 0, and d2 % 16 == 0 with
// aligned tables or any other even d2 (rotated element by element in LDS).
// ---------------------------------------------------------------------------
constexpr int kTrTile = 64;  // positions per workgroup

// In: lane (f, g) = (lane >> 3, lane & 7) holds element j = 0..7 of row f of an 8 x 8 block of
// 16-bit values (one block per g), two per register, the lower-indexed one in bits 0..15.
// Out: the same lane holds row f of the transposed block. `sel` is the byte selector of the
// first stage: 0x05040100 in lanes with even f, 0x03020706 in lanes with odd f.
__device__ __forceinline__ u32x4 transpose_8x8_halfwords(const u32x4& r, uint32_t sel)
{
    // lanes f and f ^ 1 (8 apart: a rotation by 8 inside a row of 16 lanes): afterwards register k holds
    // column 2k + (f & 1) of the row pair (f & ~1, f | 1)
    uint32_t t[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)r[k], 0x128, 0xF, 0xF, false);  // row_ror:8
        t[k] = __builtin_amdgcn_perm(other, r[k], sel);
    }
    // lanes f and f ^ 2 (16 apart): the odd rows of 16 lanes of the first register change places with the
    // even rows of the second
    const auto a = __builtin_amdgcn_permlane16_swap(t[0], t[1], false, false);
    const auto b = __builtin_amdgcn_permlane16_swap(t[2], t[3], false, false);
    // lanes f and f ^ 4 (32 apart): the upper half-wave of the first register with the lower of the second
    const auto c = __builtin_amdgcn_permlane32_swap(a[0], b[0], false, false);
    const auto d = __builtin_amdgcn_permlane32_swap(a[1], b[1], false, false);
    return u32x4{c[0], d[0], c[1], d[1]};
}

template <int DT, bool BWD, int P, typename Tables>
__global__ void __launch_bounds__(256)
rope_tr_kernel(RopeTensor T, Tables tab, int s, int cpr, int d2, int row_chunks, int64_t is_d, int rows_per_wg)
{
    static_assert(DT != NHP_F32, "16-bit data");
    constexpr int V = 8;
    constexpr bool EVAL = Tables::kEvaluate;
    extern __shared__ u32x4 tile[];  // [kTrTile][row_chunks] chunks of 8 elements
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int s0 = blockIdx.y * kTrTile;

    // Angles instead of cached tables: cos and sin of the tile's positions are evaluated once, as pairs of
    // 16-bit values behind the tile, and serve rows_per_wg (batch, head) rows; the first barrier of the
    // row loop makes them visible.
    uint32_t* const staged = reinterpret_cast<uint32_t*>(tile + kTrTile * row_chunks);  // [kTrTile][d2]
    const int rot_chunks = d2 / V;  // whole rotating chunks; d2 % 16 != 0: the rotation goes element by element
    if constexpr (EVAL) {
        for (int i = tid; i < kTrTile * d2; i += 256) {
            const int row = i / d2;
            float c = 0.0f, sn = 0.0f;
            if (s0 + row < s) tab.get(s0 + row, i - row * d2, c, sn);
            staged[i] = Half2<DT>::pack(c, sn);
        }
    }
    // cos and sin of chunk `chunk` at tile row `row` (position pos)
    auto fetch = [&](int row, int pos, int chunk, float (&c)[V], float (&sn)[V]) {
        if constexpr (EVAL) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const uint32_t w = staged[row * d2 + chunk * V + v];
                c[v] = Half2<DT>::lo(w);
                sn[v] = Half2<DT>::hi(w);
            }
        } else {
            tab.get_vec(pos, (int64_t)chunk * V, c, sn);
        }
    };
    // the same for one element
    auto fetch1 = [&](int row, int pos, int i, float& c, float& sn) {
        if constexpr (EVAL) {
            const uint32_t w = staged[row * d2 + i];
            c = Half2<DT>::lo(w);
            sn = Half2<DT>::hi(w);
        } else {
            tab.get(pos, i, c, sn);
        }
    };

    const int sc = lane & 7;  // which 8 positions of the tile
    const int f = lane >> 3;  // feature within the output chunk of this wave and pass
    const int pos8 = s0 + sc * 8;
    const uint32_t sel = (f & 1) ? 0x03020706u : 0x05040100u;
    const int half = rot_chunks / 2;

    const int r_begin = blockIdx.x * rows_per_wg;
    const int r_end = min(T.rows, r_begin + rows_per_wg);
    for (int r = r_begin; r < r_end; ++r) {
        if (r != r_begin) __syncthreads();  // the previous row's copy-out still reads the tile
        const int bi = r / T.h;
        const int hi = r - bi * T.h;
        const uint16_t* in = static_cast<const uint16_t*>(T.in) + bi * T.is_b + hi * T.is_h;
        uint16_t* out = static_cast<uint16_t*>(T.out) + bi * T.os_b + hi * T.os_h;

        u32x4 raw[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int c = p * 4 + wave;  // output chunk: wave-uniform
            raw[p] = u32x4{0, 0, 0, 0};
            if (c < cpr && pos8 < s) raw[p] = load16_stream(in + (int64_t)(c * V + f) * is_d + pos8);
        }
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int c = p * 4 + wave;
            if (c < cpr) {
                // afterwards this lane holds the 8 features of chunk c at position sc * 8 + f of the tile
                tile[(sc * 8 + f) * row_chunks + (c ^ sc)] = transpose_8x8_halfwords(raw[p], sel);
            }
        }
        __syncthreads();

        if (d2 % (2 * V) != 0) {
            // Half the rotary dimension is not a whole number of chunks (24 of 96, 20 of 80): element i pairs with
            // i + d2/2 somewhere in the middle of another chunk. The pairs are disjoint, so one work item rotates
            // up to 8 of them in place, element by element, and the tile is copied out afterwards.
            const int h2 = d2 / 2;
            const int groups = (h2 + V - 1) / V;
            for (int idx = tid; idx < kTrTile * groups; idx += 256) {
                const int row = idx / groups;
                const int i0 = (idx - row * groups) * V;
                const int pos = s0 + row;
                if (pos >= s) continue;
                const int swz = row >> 3;
                uint16_t* const base = reinterpret_cast<uint16_t*>(&tile[row * row_chunks]);
                const int cnt = (h2 - i0 < V) ? h2 - i0 : V;
                for (int e = 0; e < cnt; ++e) {
                    const int ia = i0 + e, ib = ia + h2;
                    uint16_t* const pa = base + ((((ia >> 3) ^ swz) << 3) | (ia & 7));
                    uint16_t* const pb = base + ((((ib >> 3) ^ swz) << 3) | (ib & 7));
                    float ca, sa, cb, sb;
                    fetch1(row, pos, ia, ca, sa);
                    fetch1(row, pos, ib, cb, sb);
                    const float xa = Half2<DT>::from_bits(*pa), xb = Half2<DT>::from_bits(*pb);
                    float ya, yb;
                    if (!BWD) {
                        ya = rot<DT, true>(xa, ca, xb, sa);
                        yb = rot<DT, false>(xb, cb, xa, sb);
                    } else {
                        ya = rot<DT, false>(xa, ca, xb, sb);
                        yb = rot<DT, true>(xb, cb, xa, sa);
                    }
                    *pa = Half2<DT>::to_bits(ya);
                    *pb = Half2<DT>::to_bits(yb);
                }
            }
            __syncthreads();
            for (int idx = tid; idx < kTrTile * cpr; idx += 256) {
                const int row = idx / cpr;
                const int c = idx - row * cpr;
                const int pos = s0 + row;
                if (pos >= s) continue;
                store16_stream(out + (int64_t)pos * T.os_s + (int64_t)c * V, tile[row * row_chunks + (c ^ (row >> 3))]);
            }
        } else if (rot_chunks > 0 && rot_chunks < cpr) {
            // Partial rotary dimension: rotate in place in LDS, one work item per pair of chunks (c, c + half), so
            // that every lane that does arithmetic is busy; then copy the tile out whole head vectors at a time
            // (storing the rotated chunks straight from these lanes, 32 bytes at a time, measured 20 % slower).
            // Consecutive work items take consecutive tile rows (positions) of one chunk pair: the rows of the
            // tile are 4 banks apart, so the 8 lanes of a 16-byte LDS access pass fall on distinct banks (with
            // the pair index running fastest two neighbouring rows overlapped in half of their banks).
            for (int idx = tid; idx < kTrTile * half; idx += 256) {
                const int c = idx / kTrTile;
                const int row = idx - c * kTrTile;
                const int pc = c + half;
                const int pos = s0 + row;
                if (pos >= s) continue;
                const int swz = row >> 3;
                u32x4* pa = &tile[row * row_chunks + (c ^ swz)];
                u32x4* pb = &tile[row * row_chunks + (pc ^ swz)];
                float ca[V], sa[V], cb[V], sb[V], xa[V], xb[V], ya[V], yb[V];
                fetch(row, pos, c, ca, sa);  // requesting these before the barrier, with the data, measured 3 % slower
                fetch(row, pos, pc, cb, sb);
                chunk_to_float<DT>(*pa, xa);
                chunk_to_float<DT>(*pb, xb);
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    if (!BWD) {
                        ya[v] = rot<DT, true>(xa[v], ca[v], xb[v], sa[v]);
                        yb[v] = rot<DT, false>(xb[v], cb[v], xa[v], sb[v]);
                    } else {
                        ya[v] = rot<DT, false>(xa[v], ca[v], xb[v], sb[v]);
                        yb[v] = rot<DT, true>(xb[v], cb[v], xa[v], sa[v]);
                    }
                }
                *pa = float_to_chunk<DT>(ya);
                *pb = float_to_chunk<DT>(yb);
            }
            __syncthreads();
            for (int idx = tid; idx < kTrTile * cpr; idx += 256) {
                const int row = idx / cpr;
                const int c = idx - row * cpr;
                const int pos = s0 + row;
                if (pos >= s) continue;
                store16_stream(out + (int64_t)pos * T.os_s + (int64_t)c * V, tile[row * row_chunks + (c ^ (row >> 3))]);
            }
        } else {
            for (int idx = tid; idx < kTrTile * cpr; idx += 256) {
                const int row = idx / cpr;
                const int c = idx - row * cpr;
                const int pos = s0 + row;
                if (pos >= s) continue;
                const int swz = row >> 3;
                const u32x4 x = tile[row * row_chunks + (c ^ swz)];
                u32x4 res = x;
                if (c < rot_chunks) {
                    const bool first = c < half;
                    const int pc = first ? c + half : c - half;
                    const u32x4 px = tile[row * row_chunks + (pc ^ swz)];
                    float cv[V], sv[V], unused[V], xf[V], pf[V], y[V];
                    if (!BWD) {
                        fetch(row, pos, c, cv, sv);
                    } else {
                        fetch(row, pos, c, cv, unused);
                        fetch(row, pos, pc, unused, sv);
                    }
                    const bool negate = BWD ? !first : first;
                    chunk_to_float<DT>(x, xf);
                    chunk_to_float<DT>(px, pf);
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        y[v] = negate ? rot<DT, true>(xf[v], cv[v], pf[v], sv[v]) : rot<DT>(xf[v], cv[v], pf[v], sv[v]);
                    res = float_to_chunk<DT>(y);
                }
                store16_stream(out + (int64_t)pos * T.os_s + (int64_t)c * V, res);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Scalar kernel: one thread per element, any strides, any d2.
// Index arithmetic follows fused_rotary_positional_embedding.h:27-225 of the
// reference, including odd d2 (h2 = d2/2 rounded down).
// ---------------------------------------------------------------------------
template <int DT, bool BWD, typename Tables>
__global__ void __launch_bounds__(256)
rope_scalar_kernel(void* out, const void* in, Tables tab, int64_t total, int64_t b, int64_t h, int64_t d,
                   int64_t d2, int64_t is_s, int64_t is_b, int64_t is_h, int64_t is_d, int64_t os_s,
                   int64_t os_b, int64_t os_h, int64_t os_d)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t i = idx % d;
    int64_t r = idx / d;
    const int64_t hh = r % h;
    r /= h;
    const int64_t bb = r % b;
    const int64_t pos = r / b;
    const int64_t src = pos * is_s + bb * is_b + hh * is_h;
    const int64_t dst = pos * os_s + bb * os_b + hh * os_h + i * os_d;
    const float x = Elt<DT>::load(in, src + i * is_d);
    if (i >= d2) {
        Elt<DT>::store(out, dst, x);
        return;
    }
    const int64_t h2 = d2 / 2;
    const bool first = (i + h2 < d2);
    const int64_t partner = first ? i + h2 : i + h2 - d2;
    const float xr = Elt<DT>::load(in, src + partner * is_d);
    float c, s;
    bool negate;
    if (!BWD) {
        tab.get(pos, i, c, s);
        negate = first;  // the rotated partner enters with a minus sign
    } else {
        float unused;
        tab.get(pos, i, c, unused);
        tab.get(pos, partner, unused, s);
        negate = !first;  // the shifted sine enters with a minus sign
    }
    const float res = negate ? rot<DT, true>(x, c, xr, s) : rot<DT>(x, c, xr, s);
    Elt<DT>::store(out, dst, res);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct RopeArgs {
    void* out;
    const void* in;
    int64_t s, b, h, d, d2;
    int64_t is[4], os[4];
    hipStream_t st;
};

static inline bool is_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int DT>
static bool vector_ok(const RopeArgs& a, bool tables_ok)
{
    constexpr int V = Elt<DT>::kVec;
    if (!tables_ok) return false;
    if (a.is[3] != 1 || a.os[3] != 1) return false;
    if (a.d % V != 0 || a.d2 % (2 * V) != 0 || a.d > 64 * V) return false;
    for (int i = 0; i < 3; ++i)
        if (a.is[i] % V != 0 || a.os[i] % V != 0) return false;
    if (!is_aligned16(a.in) || !is_aligned16(a.out)) return false;
    // grid.x = s workgroups of 256 threads: a grid dimension must stay below 2^32 work-items
    if (!grid_fits(a.s, 256) || a.b * a.h >= ((int64_t)1 << 30)) return false;
    return true;
}

// What rope_gather_kernel takes: the chunked layout of the vector kernels with any even rotary
// dimension and any table alignment.
template <int DT>
static bool gather_ok(const RopeArgs& a)
{
    constexpr int V = Elt<DT>::kVec;
    if (a.is[3] != 1 || a.os[3] != 1) return false;
    if (a.d % V != 0 || a.d2 % 2 != 0 || a.d2 == 0 || a.d > 64 * V) return false;
    for (int i = 0; i < 3; ++i)
        if (a.is[i] % V != 0 || a.os[i] % V != 0) return false;
    if (!is_aligned16(a.in) || !is_aligned16(a.out)) return false;
    if (!grid_fits(a.s, 256) || a.b * a.h >= ((int64_t)1 << 30)) return false;
    return true;
}

template <int DT, bool BWD, typename Tables>
static int rope_launch_scalar(const RopeArgs& a, const Tables& tab)
{
    launch_prepare();
    const int64_t total = a.s * a.b * a.h * a.d;
    const int64_t blocks = (total + 255) / 256;
    if (blocks >= ((int64_t)1 << 24)) return NHP_ERR_SHAPE;  // grid*block must stay below 2^32
    rope_scalar_kernel<DT, BWD, Tables><<<(uint32_t)blocks, 256, 0, a.st>>>(
        a.out, a.in, tab, total, a.b, a.h, a.d, a.d2, a.is[0], a.is[1], a.is[2], a.is[3], a.os[0], a.os[1],
        a.os[2], a.os[3]);
    return launch_result();
}

static RopeTensor rope_tensor(const RopeArgs& a)
{
    return RopeTensor{a.out, a.in, (int)(a.b * a.h), (int)a.h, a.is[0], a.is[1], a.is[2], a.os[0], a.os[1], a.os[2]};
}

static bool rope_flat(const RopeArgs& a) { return (a.is[1] == a.h * a.is[2]) && (a.os[1] == a.h * a.os[2]); }

// q and k as adjacent slices of one buffer: k's head vector of a row starts where q's ends, all input strides
// and all output strides agree, same batch and head counts (no grouped-query attention).
template <int DT>
static bool rope_adjacent(const RopeArgs& q, const RopeArgs& k)
{
    using S = typename Elt<DT>::storage;
    if (q.b != k.b || q.h != k.h || q.d != k.d) return false;
    if (static_cast<const S*>(k.in) != static_cast<const S*>(q.in) + q.d) return false;
    for (int i = 0; i < 3; ++i)
        if (q.is[i] != k.is[i] || q.os[i] != k.os[i]) return false;
    return 2 * q.b * q.h * (q.d / Elt<DT>::kVec) < ((int64_t)1 << 31);
}

// Launches the vector kernel for one tensor (b == nullptr) or for two tensors
// that share s, d, d2 and the tables (q and k; their head counts may differ).
// log2 of a power of two in 2..64, else -1
static int log2_chunks(int64_t cpr)
{
    for (int l = 1; l <= 6; ++l)
        if (cpr == ((int64_t)1 << l)) return l;
    return -1;
}

template <int DT, bool BWD, typename Tables>
static int rope_launch_vec(const RopeArgs& a, const RopeArgs* b, const Tables& tab)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    const int cpr = (int)(a.d / V);
    {
        const int log_cpr = log2_chunks(cpr);
        const int64_t most_rows = (b && b->b * b->h > a.b * a.h) ? b->b * b->h : a.b * a.h;
        // grid.y holds the position; row numbers inside a position are 32-bit
        if (cpr >= 2 && cpr <= 64 && a.d2 > 0 && a.s <= 65535 && most_rows * cpr < ((int64_t)1 << 31)) {
            const RopeTensor ta = rope_tensor(a);
            const RopeTensor tb = b ? rope_tensor(*b) : ta;
            const int64_t rows = most_rows;
            const bool flat = rope_flat(a) && (!b || rope_flat(*b));
            const int rot_chunks = (int)(a.d2 / V);
            if (log_cpr > 0 && log_cpr < 6 && b && rope_adjacent<DT>(a, *b)) {
                // k's head vectors lie directly behind q's: one pass over runs of 2 * cpr chunks
                const int64_t rows_per_wg = (int64_t)4 * kLeanU * (64 / (2 * cpr));
                const dim3 grid((uint32_t)((rows + rows_per_wg - 1) / rows_per_wg), (uint32_t)a.s, 1u);
#define LEAN(LC_)                                                                                             \
    case LC_:                                                                                                 \
        if (flat)                                                                                             \
            rope_lean_kernel<DT, BWD, LC_, true, Tables, true><<<grid, kLeanThreads, 0, a.st>>>(ta, tb, tab, rot_chunks, cpr);  \
        else                                                                                                  \
            rope_lean_kernel<DT, BWD, LC_, false, Tables, true><<<grid, kLeanThreads, 0, a.st>>>(ta, tb, tab, rot_chunks, cpr); \
        break;
                switch (log_cpr) {
                    LEAN(1) LEAN(2) LEAN(3) LEAN(4) LEAN(5)
                }
#undef LEAN
                return launch_result();
            }
            const int64_t rows_per_wg = (int64_t)4 * kLeanU * (64 / cpr);
            const dim3 grid((uint32_t)((rows + rows_per_wg - 1) / rows_per_wg), (uint32_t)a.s, b ? 2u : 1u);
#define LEAN(LC_)                                                                                             \
    case LC_:                                                                                                 \
        if (flat)                                                                                             \
            rope_lean_kernel<DT, BWD, LC_, true, Tables><<<grid, kLeanThreads, 0, a.st>>>(ta, tb, tab, rot_chunks, cpr);  \
        else                                                                                                  \
            rope_lean_kernel<DT, BWD, LC_, false, Tables><<<grid, kLeanThreads, 0, a.st>>>(ta, tb, tab, rot_chunks, cpr); \
        break;
            switch (log_cpr) {
                LEAN(1) LEAN(2) LEAN(3) LEAN(4) LEAN(5) LEAN(6)
            default:  // not a power of two: the chunk count is a kernel argument
                LEAN(-1)
            }
#undef LEAN
            return launch_result();
        }
    }
    const int rpw = 64 / cpr;
    const int rows_per_step = 4 * rpw;
    RopePair pair;
    pair.t[0] = rope_tensor(a);
    pair.t[1] = b ? rope_tensor(*b) : pair.t[0];
    const int rows = (b && pair.t[1].rows > pair.t[0].rows) ? pair.t[1].rows : pair.t[0].rows;
    // Workgroups per position: each makes about four steps (two unrolled loop
    // iterations) with one set of cos/sin values; measured best on MI355X.
    const int64_t steps = (rows + rows_per_step - 1) / rows_per_step;
    int64_t splits = (steps + 3) / 4;
    splits = NHP_TUNED_INT("NHP_ROPE_SPLITS", (int)splits);
    if (splits < 1) splits = 1;
    if (splits > 65535) splits = 65535;
    dim3 grid((uint32_t)a.s, (uint32_t)splits, b ? 2u : 1u);
    const bool flat = rope_flat(a) && (!b || rope_flat(*b));
    // two rows in flight per lane measured best (one is short of latency cover, four adds nothing)
    if (flat) {
        rope_vec_kernel<DT, BWD, true, 2, Tables><<<grid, 256, 0, a.st>>>(pair, tab, cpr, (int)(a.d2 / V), rpw);
    } else {
        rope_vec_kernel<DT, BWD, false, 2, Tables><<<grid, 256, 0, a.st>>>(pair, tab, cpr, (int)(a.d2 / V), rpw);
    }
    return launch_result();
}

// One tensor (b == nullptr) or q and k through rope_gather_kernel.
template <int DT, bool BWD, typename Tables>
static int rope_launch_gather(const RopeArgs& a, const RopeArgs* b, const Tables& tab)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    const int cpr = (int)(a.d / V);
    const int rpw = 64 / cpr;
    const int rows_per_step = 4 * rpw;
    RopePair pair;
    pair.t[0] = rope_tensor(a);
    pair.t[1] = b ? rope_tensor(*b) : pair.t[0];
    const int rows = (b && pair.t[1].rows > pair.t[0].rows) ? pair.t[1].rows : pair.t[0].rows;
    if (a.s <= 65535 && (int64_t)rows * cpr < ((int64_t)1 << 31)) {
        // the launch shape of the lean kernel: two rows per thread, no loop
        const int64_t rows_per_wg = (int64_t)4 * kLeanU * rpw;
        const dim3 lgrid((uint32_t)((rows + rows_per_wg - 1) / rows_per_wg), (uint32_t)a.s, b ? 2u : 1u);
        if (rope_flat(a) && (!b || rope_flat(*b)))
            rope_lean_kernel<DT, BWD, -1, true, Tables, false, true><<<lgrid, kLeanThreads, 0, a.st>>>(
                pair.t[0], pair.t[1], tab, (int)a.d2, cpr);
        else
            rope_lean_kernel<DT, BWD, -1, false, Tables, false, true><<<lgrid, kLeanThreads, 0, a.st>>>(
                pair.t[0], pair.t[1], tab, (int)a.d2, cpr);
        return launch_result();
    }
    const int64_t steps = (rows + rows_per_step - 1) / rows_per_step;
    int64_t splits = (steps + 3) / 4;  // about four steps per workgroup, as in rope_vec_kernel
    splits = NHP_TUNED_INT("NHP_ROPE_SPLITS", (int)splits);
    if (splits < 1) splits = 1;
    if (splits > 65535) splits = 65535;
    const dim3 grid((uint32_t)a.s, (uint32_t)splits, b ? 2u : 1u);
    if (rope_flat(a) && (!b || rope_flat(*b)))
        rope_gather_kernel<DT, BWD, true, 2, Tables><<<grid, 256, 0, a.st>>>(pair, tab, cpr, (int)a.d2, rpw);
    else
        rope_gather_kernel<DT, BWD, false, 2, Tables><<<grid, 256, 0, a.st>>>(pair, tab, cpr, (int)a.d2, rpw);
    return launch_result();
}

// LDS row length (in chunks) of the transposing kernel: the XOR with the load chunk index needs a
// power-of-two number of slots (at least 8), one more chunk staggers the rows over the banks.
static int tr_row_chunks(int64_t cpr)
{
    int n = 8;
    while (n < cpr) n *= 2;
    return n + 1;
}

// Dynamic LDS of the transposing kernel: the tile, and behind it the evaluated (cos, sin) pairs of its positions.
template <typename Tables>
static int64_t tr_lds_bytes(const RopeArgs& a)
{
    const int64_t tile = (int64_t)kTrTile * tr_row_chunks(a.d / 8) * 16;
    return tile + (Tables::kEvaluate ? (int64_t)kTrTile * a.d2 * 4 : 0);
}

template <int DT, typename Tables>
static bool transposed_ok(const RopeArgs& a, bool tables_ok)
{
    if (DT == NHP_F32) return false;
    // whole rotating chunks are fetched from the tables 16 bytes at a time; otherwise element by element
    if (a.d2 % 16 == 0 ? !tables_ok : a.d2 % 2 != 0) return false;
    if (tr_lds_bytes<Tables>(a) > 65536) return false;
    if (a.is[0] != 1 || a.os[3] != 1 || a.is[3] % 8 != 0) return false;
    if (a.s % 8 != 0 || a.d % 8 != 0 || a.d > 256) return false;
    const int64_t passes = (a.d + 31) / 32;
    if (passes != 2 && passes != 3 && passes != 4 && passes != 8) return false;
    if (a.is[1] % 8 != 0 || a.is[2] % 8 != 0) return false;
    for (int i = 0; i < 3; ++i)
        if (a.os[i] % 8 != 0) return false;
    if (!is_aligned16(a.in) || !is_aligned16(a.out)) return false;
    if (a.b * a.h >= ((int64_t)1 << 31) || (a.s + kTrTile - 1) / kTrTile > 65535) return false;
    return true;
}

template <int DT, bool BWD, typename Tables>
static int rope_launch_transposed(const RopeArgs& a, const Tables& tab)
{
    launch_prepare();
    if constexpr (DT == NHP_F32) {
        return NHP_ERR_SHAPE;
    } else {
        const int cpr = (int)(a.d / 8);
        const int row_chunks = tr_row_chunks(cpr);
        const uint32_t lds = (uint32_t)tr_lds_bytes<Tables>(a);
        const int64_t rows = a.b * a.h, tiles = (a.s + kTrTile - 1) / kTrTile;
        // Evaluated tables are shared by several rows per workgroup, as many as leave about a thousand
        // workgroups (at most 8); cached tables: one row per workgroup.
        int rows_per_wg = 1;
        if (Tables::kEvaluate) {
            const int64_t want = rows * tiles / 1024;
            rows_per_wg = (int)(want < 1 ? 1 : want > 8 ? 8 : want);
        }
        const dim3 grid((uint32_t)((rows + rows_per_wg - 1) / rows_per_wg), (uint32_t)tiles);
        const RopeTensor t = rope_tensor(a);
#define CASE(P_)                                                                                              \
    case P_:                                                                                                  \
        rope_tr_kernel<DT, BWD, P_, Tables><<<grid, 256, lds, a.st>>>(t, tab, (int)a.s, cpr, (int)a.d2,         \
                                                                      row_chunks, a.is[3], rows_per_wg);      \
        break;
        switch ((int)((a.d + 31) / 32)) {
            CASE(2) CASE(3) CASE(4) CASE(8)
        default:
            return NHP_ERR_SHAPE;
        }
#undef CASE
        return launch_result();
    }
}

template <int DT, bool BWD, typename Tables>
static int rope_launch(const RopeArgs& a, const Tables& tab, bool tables_ok)
{
    if (vector_ok<DT>(a, tables_ok)) return rope_launch_vec<DT, BWD>(a, nullptr, tab);
    if (transposed_ok<DT, Tables>(a, tables_ok)) return rope_launch_transposed<DT, BWD>(a, tab);
    if (gather_ok<DT>(a)) return rope_launch_gather<DT, BWD>(a, nullptr, tab);
    return rope_launch_scalar<DT, BWD>(a, tab);
}

// q and k in one launch when both qualify for the vector kernel, otherwise one launch each.
template <int DT, bool BWD, typename Tables>
static int rope_launch_pair(const RopeArgs& q, const RopeArgs& k, const Tables& tab, bool tables_ok)
{
    if (vector_ok<DT>(q, tables_ok) && vector_ok<DT>(k, tables_ok)) return rope_launch_vec<DT, BWD>(q, &k, tab);
    if (!vector_ok<DT>(q, tables_ok) && !vector_ok<DT>(k, tables_ok) && gather_ok<DT>(q) && gather_ok<DT>(k) &&
        !transposed_ok<DT, Tables>(q, tables_ok) && !transposed_ok<DT, Tables>(k, tables_ok))
        return rope_launch_gather<DT, BWD>(q, &k, tab);
    const int rc = rope_launch<DT, BWD>(q, tab, tables_ok);
    if (rc != NHP_OK) return rc;
    return rope_launch<DT, BWD>(k, tab, tables_ok);
}

static int check_common(const void* out, const void* in, int64_t s, int64_t b, int64_t h, int64_t d,
                        int64_t d2, const int64_t* is, const int64_t* os, bool& empty)
{
    empty = false;
    if (s < 0 || b < 0 || h < 0 || d < 0 || d2 < 0 || d2 > d) return NHP_ERR_SHAPE;
    if (!is || !os) return NHP_ERR_NULL;
    if (s == 0 || b == 0 || h == 0 || d == 0) {
        empty = true;
        return NHP_OK;
    }
    if (!out || !in) return NHP_ERR_NULL;
    if (out == in) return NHP_ERR_ALIAS;
    return NHP_OK;
}

template <bool BWD>
static int rope_cached(void* out, const void* in, const void* cos, const void* sin, int64_t s, int64_t b,
                       int64_t h, int64_t d, int64_t d2, const int64_t* is, const int64_t* os, int dtype,
                       int cs_dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    if (cs_dtype != NHP_F32 && cs_dtype != dtype) return NHP_ERR_DTYPE;
    bool empty;
    const int rc = check_common(out, in, s, b, h, d, d2, is, os, empty);
    if (rc != NHP_OK || empty) return rc;
    if (d2 > 0 && (!cos || !sin)) return NHP_ERR_NULL;
    RopeArgs a{out, in, s, b, h, d, d2, {is[0], is[1], is[2], is[3]}, {os[0], os[1], os[2], os[3]},
               static_cast<hipStream_t>(stream)};
    const int cs_size = (cs_dtype == NHP_F32) ? 4 : 2;
    const bool tab_ok = is_aligned16(cos) && is_aligned16(sin) && (d2 * cs_size) % 16 == 0;
#define NHP_ROPE_CASE(DT_, CS_)                                         \
    if (dtype == DT_ && cs_dtype == CS_) {                              \
        CachedTables<DT_, CS_> tab{cos, sin, d2};                       \
        return rope_launch<DT_, BWD>(a, tab, tab_ok);                   \
    }
    NHP_ROPE_CASE(NHP_BF16, NHP_BF16)
    NHP_ROPE_CASE(NHP_BF16, NHP_F32)
    NHP_ROPE_CASE(NHP_F16, NHP_F16)
    NHP_ROPE_CASE(NHP_F16, NHP_F32)
    NHP_ROPE_CASE(NHP_F32, NHP_F32)
#undef NHP_ROPE_CASE
    return NHP_ERR_DTYPE;
}

template <bool BWD>
static int rope_freqs(void* out, const void* in, const float* freqs, int64_t s, int64_t b, int64_t h,
                      int64_t d, int64_t d2, const int64_t* is, const int64_t* os, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    bool empty;
    const int rc = check_common(out, in, s, b, h, d, d2, is, os, empty);
    if (rc != NHP_OK || empty) return rc;
    if (d2 > 0 && !freqs) return NHP_ERR_NULL;
    RopeArgs a{out, in, s, b, h, d, d2, {is[0], is[1], is[2], is[3]}, {os[0], os[1], os[2], os[3]},
               static_cast<hipStream_t>(stream)};
    if (dtype == NHP_BF16) return rope_launch<NHP_BF16, BWD>(a, FreqTable<NHP_BF16>{freqs, d2}, true);
    if (dtype == NHP_F16) return rope_launch<NHP_F16, BWD>(a, FreqTable<NHP_F16>{freqs, d2}, true);
    return rope_launch<NHP_F32, BWD>(a, FreqTable<NHP_F32>{freqs, d2}, true);
}

template <bool BWD>
static int rope_cached_qk(void* q_out, void* k_out, const void* q_in, const void* k_in, const void* cos,
                          const void* sin, int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                          const int64_t* qis, const int64_t* kis, const int64_t* qos, const int64_t* kos, int dtype,
                          int cs_dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    if (cs_dtype != NHP_F32 && cs_dtype != dtype) return NHP_ERR_DTYPE;
    bool empty_q, empty_k;
    int rc = check_common(q_out, q_in, s, b, hq, d, d2, qis, qos, empty_q);
    if (rc != NHP_OK) return rc;
    rc = check_common(k_out, k_in, s, b, hk, d, d2, kis, kos, empty_k);
    if (rc != NHP_OK) return rc;
    if (empty_q || empty_k) {
        // at most one tensor has work: hand it to the single-tensor path
        if (!empty_q)
            return rope_cached<BWD>(q_out, q_in, cos, sin, s, b, hq, d, d2, qis, qos, dtype, cs_dtype, stream);
        if (!empty_k)
            return rope_cached<BWD>(k_out, k_in, cos, sin, s, b, hk, d, d2, kis, kos, dtype, cs_dtype, stream);
        return NHP_OK;
    }
    if (q_out == k_in || k_out == q_in || q_out == k_out) return NHP_ERR_ALIAS;
    if (d2 > 0 && (!cos || !sin)) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    RopeArgs q{q_out, q_in, s, b, hq, d, d2, {qis[0], qis[1], qis[2], qis[3]}, {qos[0], qos[1], qos[2], qos[3]}, st};
    RopeArgs k{k_out, k_in, s, b, hk, d, d2, {kis[0], kis[1], kis[2], kis[3]}, {kos[0], kos[1], kos[2], kos[3]}, st};
    const int cs_size = (cs_dtype == NHP_F32) ? 4 : 2;
    const bool tab_ok = is_aligned16(cos) && is_aligned16(sin) && (d2 * cs_size) % 16 == 0;
#define NHP_ROPE_CASE(DT_, CS_)                                         \
    if (dtype == DT_ && cs_dtype == CS_) {                              \
        CachedTables<DT_, CS_> tab{cos, sin, d2};                       \
        return rope_launch_pair<DT_, BWD>(q, k, tab, tab_ok);           \
    }
    NHP_ROPE_CASE(NHP_BF16, NHP_BF16)
    NHP_ROPE_CASE(NHP_BF16, NHP_F32)
    NHP_ROPE_CASE(NHP_F16, NHP_F16)
    NHP_ROPE_CASE(NHP_F16, NHP_F32)
    NHP_ROPE_CASE(NHP_F32, NHP_F32)
#undef NHP_ROPE_CASE
    return NHP_ERR_DTYPE;
}

template <bool BWD>
static int rope_freqs_qk(void* q_out, void* k_out, const void* q_in, const void* k_in, const float* freqs, int64_t s,
                         int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2, const int64_t* qis,
                         const int64_t* kis, const int64_t* qos, const int64_t* kos, int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    bool empty_q, empty_k;
    int rc = check_common(q_out, q_in, s, b, hq, d, d2, qis, qos, empty_q);
    if (rc != NHP_OK) return rc;
    rc = check_common(k_out, k_in, s, b, hk, d, d2, kis, kos, empty_k);
    if (rc != NHP_OK) return rc;
    if (empty_q || empty_k) {
        if (!empty_q) return rope_freqs<BWD>(q_out, q_in, freqs, s, b, hq, d, d2, qis, qos, dtype, stream);
        if (!empty_k) return rope_freqs<BWD>(k_out, k_in, freqs, s, b, hk, d, d2, kis, kos, dtype, stream);
        return NHP_OK;
    }
    if (q_out == k_in || k_out == q_in || q_out == k_out) return NHP_ERR_ALIAS;
    if (d2 > 0 && !freqs) return NHP_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    RopeArgs q{q_out, q_in, s, b, hq, d, d2, {qis[0], qis[1], qis[2], qis[3]}, {qos[0], qos[1], qos[2], qos[3]}, st};
    RopeArgs k{k_out, k_in, s, b, hk, d, d2, {kis[0], kis[1], kis[2], kis[3]}, {kos[0], kos[1], kos[2], kos[3]}, st};
    if (dtype == NHP_BF16) return rope_launch_pair<NHP_BF16, BWD>(q, k, FreqTable<NHP_BF16>{freqs, d2}, true);
    if (dtype == NHP_F16) return rope_launch_pair<NHP_F16, BWD>(q, k, FreqTable<NHP_F16>{freqs, d2}, true);
    return rope_launch_pair<NHP_F32, BWD>(q, k, FreqTable<NHP_F32>{freqs, d2}, true);
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int nhp_rope_cached_fwd(void* out, const void* in, const void* cos, const void* sin, int64_t s, int64_t b,
                        int64_t h, int64_t d, int64_t d2, const int64_t in_stride[4],
                        const int64_t out_stride[4], int dtype, int cs_dtype, void* stream)
{
    return rope_cached<false>(out, in, cos, sin, s, b, h, d, d2, in_stride, out_stride, dtype, cs_dtype,
                              stream);
}

int nhp_rope_cached_bwd(void* out, const void* in, const void* cos, const void* sin, int64_t s, int64_t b,
                        int64_t h, int64_t d, int64_t d2, const int64_t in_stride[4],
                        const int64_t out_stride[4], int dtype, int cs_dtype, void* stream)
{
    return rope_cached<true>(out, in, cos, sin, s, b, h, d, d2, in_stride, out_stride, dtype, cs_dtype,
                             stream);
}

int nhp_rope_freqs_fwd(void* out, const void* in, const float* freqs, int64_t s, int64_t b, int64_t h,
                       int64_t d, int64_t d2, const int64_t in_stride[4], const int64_t out_stride[4],
                       int dtype, void* stream)
{
    return rope_freqs<false>(out, in, freqs, s, b, h, d, d2, in_stride, out_stride, dtype, stream);
}

int nhp_rope_freqs_bwd(void* out, const void* in, const float* freqs, int64_t s, int64_t b, int64_t h,
                       int64_t d, int64_t d2, const int64_t in_stride[4], const int64_t out_stride[4],
                       int dtype, void* stream)
{
    return rope_freqs<true>(out, in, freqs, s, b, h, d, d2, in_stride, out_stride, dtype, stream);
}

int nhp_rope_cached_qk_fwd(void* q_out, void* k_out, const void* q_in, const void* k_in, const void* cos,
                           const void* sin, int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                           const int64_t q_in_stride[4], const int64_t k_in_stride[4],
                           const int64_t q_out_stride[4], const int64_t k_out_stride[4], int dtype, int cs_dtype,
                           void* stream)
{
    return rope_cached_qk<false>(q_out, k_out, q_in, k_in, cos, sin, s, b, hq, hk, d, d2, q_in_stride, k_in_stride,
                                 q_out_stride, k_out_stride, dtype, cs_dtype, stream);
}

int nhp_rope_cached_qk_bwd(void* q_out, void* k_out, const void* q_in, const void* k_in, const void* cos,
                           const void* sin, int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                           const int64_t q_in_stride[4], const int64_t k_in_stride[4],
                           const int64_t q_out_stride[4], const int64_t k_out_stride[4], int dtype, int cs_dtype,
                           void* stream)
{
    return rope_cached_qk<true>(q_out, k_out, q_in, k_in, cos, sin, s, b, hq, hk, d, d2, q_in_stride, k_in_stride,
                                q_out_stride, k_out_stride, dtype, cs_dtype, stream);
}

int nhp_rope_freqs_qk_fwd(void* q_out, void* k_out, const void* q_in, const void* k_in, const float* freqs, int64_t s,
                          int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2, const int64_t q_in_stride[4],
                          const int64_t k_in_stride[4], const int64_t q_out_stride[4], const int64_t k_out_stride[4],
                          int dtype, void* stream)
{
    return rope_freqs_qk<false>(q_out, k_out, q_in, k_in, freqs, s, b, hq, hk, d, d2, q_in_stride, k_in_stride,
                                q_out_stride, k_out_stride, dtype, stream);
}

int nhp_rope_freqs_qk_bwd(void* q_out, void* k_out, const void* q_in, const void* k_in, const float* freqs, int64_t s,
                          int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2, const int64_t q_in_stride[4],
                          const int64_t k_in_stride[4], const int64_t q_out_stride[4], const int64_t k_out_stride[4],
                          int dtype, void* stream)
{
    return rope_freqs_qk<true>(q_out, k_out, q_in, k_in, freqs, s, b, hq, hk, d, d2, q_in_stride, k_in_stride,
                               q_out_stride, k_out_stride, dtype, stream);
}

int nhp_abi_version(void) { return 1; }

const char* nhp_status_string(int status)
{
    switch (status) {
        case NHP_OK: return "ok";
        case NHP_ERR_DTYPE: return "unsupported dtype";
        case NHP_ERR_SHAPE: return "invalid or unsupported shape";
        case NHP_ERR_NULL: return "null pointer for a non-empty tensor";
        case NHP_ERR_PAD_BATCHES: return "mask batch dimension must be 1 or equal to the batch size";
        case NHP_ERR_LAUNCH: return "kernel launch failed";
        case NHP_ERR_ALIAS: return "output aliases an input";
        case NHP_ERR_SCRATCH: return "input needs more scratch memory than the entry point's fixed buffer holds";
        default: return "unknown status";
    }
}

}  // extern "C"
