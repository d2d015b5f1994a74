// Device-side helpers shared by all kernels of the library (gfx950, wave64).
//
// Everything here assumes a 64-lane wavefront and is compiled for gfx950 only.
// The translation units are built with -ffp-contract=off: a fused multiply-add
// appears only where the source says fmaf().
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/neox_hotpath.h"

namespace nhp {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -__builtin_huge_valf();

template <typename To, typename From>
__device__ __forceinline__ To bitcast(From v)
{
    return __builtin_bit_cast(To, v);
}

// ---------------------------------------------------------------------------
// 16-bit storage formats. A 32-bit word holds two consecutive elements, the
// lower-addressed one in bits 0..15.
// ---------------------------------------------------------------------------
template <int DT>
struct Half2;

template <>
struct Half2<NHP_BF16> {
    static __device__ __forceinline__ float lo(uint32_t w) { return bitcast<float>(w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return bitcast<float>(w & 0xffff0000u); }
    // round-to-nearest-even, v_cvt_pk_bf16_f32 on gfx950
    static __device__ __forceinline__ uint32_t pack(float a, float b)
    {
        f32x2 v = {a, b};
        return bitcast<uint32_t>(__builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ float round(float a)
    {
        return (float)(__bf16)a;
    }
    static __device__ __forceinline__ float from_bits(uint16_t h)
    {
        return bitcast<float>((uint32_t)h << 16);
    }
    static __device__ __forceinline__ uint16_t to_bits(float a)
    {
        return bitcast<uint16_t>((__bf16)a);
    }
};

template <>
struct Half2<NHP_F16> {
    static __device__ __forceinline__ float lo(uint32_t w) { return (float)bitcast<f16x2>(w)[0]; }
    static __device__ __forceinline__ float hi(uint32_t w) { return (float)bitcast<f16x2>(w)[1]; }
    // round-to-nearest-even (the wave's default rounding mode), v_cvt_pk_f16_f32
    static __device__ __forceinline__ uint32_t pack(float a, float b)
    {
        f32x2 v = {a, b};
        return bitcast<uint32_t>(__builtin_convertvector(v, f16x2));
    }
    static __device__ __forceinline__ float round(float a)
    {
        return (float)(_Float16)a;
    }
    static __device__ __forceinline__ float from_bits(uint16_t h)
    {
        return (float)bitcast<_Float16>(h);
    }
    static __device__ __forceinline__ uint16_t to_bits(float a)
    {
        return bitcast<uint16_t>((_Float16)a);
    }
};

// Two values rounded to the storage type with one packed conversion (three instructions for the pair
// instead of four).
template <int DT>
__device__ __forceinline__ void round_pair(float& a, float& b)
{
    const uint32_t w = Half2<DT>::pack(a, b);
    a = Half2<DT>::lo(w);
    b = Half2<DT>::hi(w);
}

// Unpack the eight elements of a 16-byte chunk.
template <int DT>
__device__ __forceinline__ void unpack8(const u32x4& raw, float (&f)[8])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = Half2<DT>::lo(raw[i]);
        f[2 * i + 1] = Half2<DT>::hi(raw[i]);
    }
}

template <int DT>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8])
{
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = Half2<DT>::pack(f[2 * i], f[2 * i + 1]);
    return r;
}

// ---------------------------------------------------------------------------
// Element types (the two 16-bit formats and fp32) behind one interface; a
// 16-byte chunk holds kVec elements.
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

// ---------------------------------------------------------------------------
// Streaming global memory access: every byte of these tensors is touched once,
// so loads and stores carry the non-temporal hint.
// ---------------------------------------------------------------------------
__device__ __forceinline__ u32x4 load16_stream(const void* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void store16_stream(void* p, u32x4 v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ u32x4 load16(const void* p)
{
    return *reinterpret_cast<const u32x4*>(p);
}
__device__ __forceinline__ u32x2 load8(const void* p)
{
    return *reinterpret_cast<const u32x2*>(p);
}

// ---------------------------------------------------------------------------
// Cross-lane reductions over groups of L consecutive lanes (L a power of two,
// 1..64). Lanes 2^k apart are combined with DPP controls inside a row of 16
// lanes, ds_swizzle for the 16<->16 exchange and v_readlane for the two
// halves of the wave. Every lane of the group ends up with the group result.
// ---------------------------------------------------------------------------
struct OpMax {
    static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
};
struct OpSum {
    static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
    return bitcast<float>(
        __builtin_amdgcn_update_dpp(0, bitcast<int>(v), CTRL, 0xF, 0xF, true));
}

template <typename Op, int L>
__device__ __forceinline__ float group_reduce(float v)
{
    static_assert(L >= 1 && L <= 64 && (L & (L - 1)) == 0, "L must be a power of two <= 64");
    if constexpr (L >= 2) v = Op::apply(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    if constexpr (L >= 4) v = Op::apply(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    if constexpr (L >= 8) v = Op::apply(v, dpp_move<0x141>(v));  // row_half_mirror
    if constexpr (L >= 16) v = Op::apply(v, dpp_move<0x140>(v)); // row_mirror
    if constexpr (L >= 32) {
        // swap lanes i and i^16 (bit-mode swizzle: and 0x1f, or 0, xor 0x10)
        v = Op::apply(v, bitcast<float>(__builtin_amdgcn_ds_swizzle(bitcast<int>(v), 0x401F)));
    }
    if constexpr (L >= 64) {
        float a = bitcast<float>(__builtin_amdgcn_readlane(bitcast<int>(v), 0));
        float b = bitcast<float>(__builtin_amdgcn_readlane(bitcast<int>(v), 32));
        v = Op::apply(a, b);
    }
    return v;
}

// Combine the per-wave partials of the W waves of a workgroup through LDS.
// `slots` must hold at least W floats and must not be reused for another
// reduction before a later barrier.
template <typename Op, int W>
__device__ __forceinline__ float block_combine(float v, float* slots, int wave, int lane)
{
    if constexpr (W == 1) {
        return v;
    } else {
        if (lane == 0) slots[wave] = v;
        __syncthreads();
        float r = slots[0];
#pragma unroll
        for (int i = 1; i < W; ++i) r = Op::apply(r, slots[i]);
        return r;
    }
}

// 2^(x) with the raw v_exp_f32 instruction (about 1 ulp, no denormal results).
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------
// Counter-based random bits for dropout masks
// ---------------------------------------------------------------------------
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11)
struct Philox {
    uint32_t v[4];
};

__device__ __forceinline__ Philox philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                uint32_t k1)
{
    constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        // one 32 x 32 -> 64 bit multiply per product (v_mad_u64_u32) instead of a high and a low one
        const uint64_t p0 = (uint64_t)M0 * c0, p1 = (uint64_t)M1 * c2;
        const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
        const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
        const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
        c0 = n0;
        c1 = lo1;
        c2 = n2;
        c3 = lo0;
        k0 += W0;
        k1 += W1;
    }
    return Philox{{c0, c1, c2, c3}};
}

// 16-bit random value of element `lane8` (0..7) of the group of eight elements `group`
__device__ __forceinline__ uint32_t random16(const Philox& r, int lane8)
{
    return (r.v[lane8 >> 1] >> ((lane8 & 1) * 16)) & 0xffffu;
}

// Dropout parameters as the kernels take them: keep when random16 < threshold, kept values are
// multiplied by scale = 1 / (1 - p); counter = (element index / 8, offset), key = seed.
struct DropoutKey {
    uint32_t threshold;
    float scale;
    uint32_t seed_lo, seed_hi, off_lo, off_hi;
};

// Random bits for the group of eight consecutive elements that starts at flat index e0 (a multiple of 8).
__device__ __forceinline__ Philox dropout_bits(const DropoutKey& k, uint64_t e0)
{
    const uint64_t group = e0 >> 3;
    return philox4x32_10((uint32_t)group, (uint32_t)(group >> 32), k.off_lo, k.off_hi, k.seed_lo, k.seed_hi);
}

static inline DropoutKey make_dropout_key(float p, uint64_t seed, uint64_t offset)
{
    DropoutKey k;
    const double keep = 1.0 - (double)p;
    const uint32_t threshold = (uint32_t)(keep * 65536.0 + 0.5);
    k.threshold = threshold > 65536u ? 65536u : threshold;
    k.scale = (float)(1.0 / keep);
    k.seed_lo = (uint32_t)seed;
    k.seed_hi = (uint32_t)(seed >> 32);
    k.off_lo = (uint32_t)offset;
    k.off_hi = (uint32_t)(offset >> 32);
    return k;
}

// ---------------------------------------------------------------------------
// Launch-shape constants are written as NHP_TUNED_INT("NAME", default). This library
// always takes the default; an experimental build can pre-include a header that
// defines the macro differently (compiler option -include) to sweep the values.
// ---------------------------------------------------------------------------
#ifndef NHP_TUNED_INT
#define NHP_TUNED_INT(name, def) (def)
#endif

// ---------------------------------------------------------------------------
// Host-side launch checks
// ---------------------------------------------------------------------------
static inline bool ptr_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
// A grid of `blocks` workgroups of `threads` work-items must stay below 2^32 work-items.
static inline bool grid_fits(int64_t blocks, int threads) { return blocks > 0 && blocks * threads < ((int64_t)1 << 32); }
// hipGetLastError() returns and clears whatever error is pending on the calling thread, also one
// left by an earlier call of the application's. launch_prepare() clears such a leftover before the
// first launch of an entry point, so that launch_result() reports this library's launches only.
static inline void launch_prepare() { (void)hipGetLastError(); }
static inline int launch_result() { return hipGetLastError() == hipSuccess ? NHP_OK : NHP_ERR_LAUNCH; }

}  // namespace nhp
