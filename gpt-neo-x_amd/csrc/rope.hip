// Fused rotary positional embedding (rotate-half form), forward and backward,
// for gfx950.
//
// Tensor t is [s, b, h, d] with arbitrary element strides; the first d2
// elements of every head vector are rotated with the angle of position s,
// the remaining d - d2 are copied.
//
// Vector kernel. A head vector is cut into 16-byte chunks (V = 8 elements for
// 16-bit data, 4 for fp32). The rotation pairs element i with i + d2/2, so a
// lane takes the two chunks [i, i+V) and [i+d2/2, i+d2/2+V) together: every
// element is loaded once and no data crosses lanes. The pass-through tail is
// cut into units of two chunks as well. A head vector is thus U units wide and
// a workgroup is laid out as [heads][U] for one sequence position; it walks
// over a slice of the batch dimension re-using the cos/sin values it loaded
// (or computed) once.
//
// Arithmetic: out = (x (*) c) (+) (r (*) s) where every product and the sum
// are rounded to the data dtype, which is what the scalar types of the
// reference kernels and eager torch do.

#include "common.hpp"

namespace nhp {

// ---------------------------------------------------------------------------
// element types
// ---------------------------------------------------------------------------
template <int DT>
struct Elt;

template <>
struct Elt<NHP_BF16> {
    using storage = uint16_t;
    static constexpr int kVec = 8;
    static __device__ __forceinline__ float load(const void* p, int64_t i)
    {
        return Half2<NHP_BF16>::from_bits(static_cast<const uint16_t*>(p)[i]);
    }
    static __device__ __forceinline__ void store(void* p, int64_t i, float v)
    {
        static_cast<uint16_t*>(p)[i] = Half2<NHP_BF16>::to_bits(v);
    }
    static __device__ __forceinline__ float round(float v) { return Half2<NHP_BF16>::round(v); }
};
template <>
struct Elt<NHP_F16> {
    using storage = uint16_t;
    static constexpr int kVec = 8;
    static __device__ __forceinline__ float load(const void* p, int64_t i)
    {
        return Half2<NHP_F16>::from_bits(static_cast<const uint16_t*>(p)[i]);
    }
    static __device__ __forceinline__ void store(void* p, int64_t i, float v)
    {
        static_cast<uint16_t*>(p)[i] = Half2<NHP_F16>::to_bits(v);
    }
    static __device__ __forceinline__ float round(float v) { return Half2<NHP_F16>::round(v); }
};
template <>
struct Elt<NHP_F32> {
    using storage = float;
    static constexpr int kVec = 4;
    static __device__ __forceinline__ float load(const void* p, int64_t i)
    {
        return static_cast<const float*>(p)[i];
    }
    static __device__ __forceinline__ void store(void* p, int64_t i, float v)
    {
        static_cast<float*>(p)[i] = v;
    }
    static __device__ __forceinline__ float round(float v) { return v; }
};

// A 16-byte chunk as V floats.
template <int DT>
__device__ __forceinline__ void chunk_to_float(const u32x4& raw, float (&f)[Elt<DT>::kVec])
{
    if constexpr (DT == NHP_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = bitcast<float>(raw[i]);
    } else {
        unpack8<DT>(raw, f);
    }
}
template <int DT>
__device__ __forceinline__ u32x4 float_to_chunk(const float (&f)[Elt<DT>::kVec])
{
    if constexpr (DT == NHP_F32) {
        return u32x4{bitcast<uint32_t>(f[0]), bitcast<uint32_t>(f[1]), bitcast<uint32_t>(f[2]),
                     bitcast<uint32_t>(f[3])};
    } else {
        return pack8<DT>(f);
    }
}

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

// ---------------------------------------------------------------------------
// Vector kernel
//   grid  = (s, ceil(b / b_per_block)), block = heads_per_block * U threads (<= 256)
//   unit u < np : rotary pair of chunks  i = u*V  and  i + h2
//   unit u >= np: tail chunks 2*(u-np) and 2*(u-np)+1 (the second may not exist)
// Requires: stride_d == 1 on both sides, d2 % (2V) == 0, (d-d2) % V == 0,
// every other stride a multiple of V, 16-byte aligned base pointers.
// ---------------------------------------------------------------------------
template <int DT, bool BWD, typename Tables>
__global__ void __launch_bounds__(256)
rope_vec_kernel(void* out, const void* in, Tables tab, int b, int h, int d, int d2, int units,
                int heads_per_block, int b_per_block, int64_t is_s, int64_t is_b, int64_t is_h,
                int64_t os_s, int64_t os_b, int64_t os_h)
{
    constexpr int V = Elt<DT>::kVec;
    using S = typename Elt<DT>::storage;
    const int u = threadIdx.x % units;
    const int hl = threadIdx.x / units;
    if (hl >= heads_per_block) return;
    const int64_t pos = blockIdx.x;
    const int h2 = d2 / 2;
    const int np = h2 / V;  // rotary units per head vector
    const int b0 = blockIdx.y * b_per_block;
    const int b1 = (b0 + b_per_block < b) ? b0 + b_per_block : b;

    const S* ip = static_cast<const S*>(in) + pos * is_s;
    S* op = static_cast<S*>(out) + pos * os_s;

    if (u < np) {
        const int i = u * V;
        float ca[V], sa[V], cb[V], sb[V];
        tab.get_vec(pos, i, ca, sa);
        tab.get_vec(pos, i + h2, cb, sb);
        for (int hh = hl; hh < h; hh += heads_per_block) {
            for (int bb = b0; bb < b1; ++bb) {
                const S* src = ip + bb * is_b + hh * is_h;
                S* dst = op + bb * os_b + hh * os_h;
                float xa[V], xb[V], ya[V], yb[V];
                chunk_to_float<DT>(load16_stream(src + i), xa);
                chunk_to_float<DT>(load16_stream(src + i + h2), xb);
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    if (!BWD) {
                        // y_a = x_a*c_a + (-x_b)*s_a ; y_b = x_b*c_b + x_a*s_b
                        ya[v] = rot<DT, true>(xa[v], ca[v], xb[v], sa[v]);
                        yb[v] = rot<DT>(xb[v], cb[v], xa[v], sb[v]);
                    } else {
                        // dx_a = g_a*c_a + g_b*s_b ; dx_b = g_b*c_b + g_a*(-s_a)
                        ya[v] = rot<DT>(xa[v], ca[v], xb[v], sb[v]);
                        yb[v] = rot<DT, true>(xb[v], cb[v], xa[v], sa[v]);
                    }
                }
                store16_stream(dst + i, float_to_chunk<DT>(ya));
                store16_stream(dst + i + h2, float_to_chunk<DT>(yb));
            }
        }
    } else {
        const int c0 = d2 + 2 * (u - np) * V;
        const bool second = c0 + V < d;
        for (int hh = hl; hh < h; hh += heads_per_block) {
            for (int bb = b0; bb < b1; ++bb) {
                const S* src = ip + bb * is_b + hh * is_h;
                S* dst = op + bb * os_b + hh * os_h;
                const u32x4 a = load16_stream(src + c0);
                u32x4 c = u32x4{0, 0, 0, 0};
                if (second) c = load16_stream(src + c0 + V);
                store16_stream(dst + c0, a);
                if (second) store16_stream(dst + c0 + V, c);
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
    if (a.d2 % (2 * V) != 0 || (a.d - a.d2) % V != 0) return false;
    for (int i = 0; i < 3; ++i)
        if (a.is[i] % V != 0 || a.os[i] % V != 0) return false;
    if (!is_aligned16(a.in) || !is_aligned16(a.out)) return false;
    const int64_t units = a.d2 / (2 * V) + ((a.d - a.d2) / V + 1) / 2;
    if (units > 256) return false;
    if (a.s >= ((int64_t)1 << 31) || a.b > 65535 * (int64_t)64 || a.h >= ((int64_t)1 << 30)) return false;
    return true;
}

template <int DT, bool BWD, typename Tables>
static int rope_launch(const RopeArgs& a, const Tables& tab, bool tables_ok)
{
    constexpr int V = Elt<DT>::kVec;
    if (vector_ok<DT>(a, tables_ok)) {
        const int units = (int)(a.d2 / (2 * V) + ((a.d - a.d2) / V + 1) / 2);
        int hpb = 256 / units;
        if (hpb > a.h) hpb = (int)a.h;
        // batch entries per workgroup: re-use cos/sin over a few of them, but
        // keep at least ~16 workgroups per CU in the grid
        int bpb = 1;
        const int64_t head_passes = (a.h + hpb - 1) / hpb;
        while (bpb * 2 <= a.b && bpb * head_passes < 4 &&
               a.s * ((a.b + bpb * 2 - 1) / (bpb * 2)) >= 4096)
            bpb *= 2;
        const int64_t gy = (a.b + bpb - 1) / bpb;
        if (gy > 65535) return NHP_ERR_SHAPE;
        dim3 grid((uint32_t)a.s, (uint32_t)gy);
        rope_vec_kernel<DT, BWD, Tables><<<grid, hpb * units, 0, a.st>>>(
            a.out, a.in, tab, (int)a.b, (int)a.h, (int)a.d, (int)a.d2, units, hpb, bpb, a.is[0], a.is[1],
            a.is[2], a.os[0], a.os[1], a.os[2]);
    } else {
        const int64_t total = a.s * a.b * a.h * a.d;
        const int64_t blocks = (total + 255) / 256;
        if (blocks >= ((int64_t)1 << 24)) return NHP_ERR_SHAPE;  // grid*block must stay below 2^32
        rope_scalar_kernel<DT, BWD, Tables><<<(uint32_t)blocks, 256, 0, a.st>>>(
            a.out, a.in, tab, total, a.b, a.h, a.d, a.d2, a.is[0], a.is[1], a.is[2], a.is[3], a.os[0],
            a.os[1], a.os[2], a.os[3]);
    }
    return hipGetLastError() == hipSuccess ? NHP_OK : NHP_ERR_LAUNCH;
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
        default: return "unknown status";
    }
}

}  // extern "C"
