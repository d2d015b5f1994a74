// Gated MLP activations (SwiGLU, GeGLU, ReGLU, GLU, bilinear) for gfx950,
// forward and backward.
//
// The input is [rows, 2 * F]: the first F features of a row are the values x,
// the last F the gates g (what chunk(2, dim=-1) returns); with a bias [2 * F]
// both halves get their half of it. out[rows, F] = act(g) * x.
//
// Same launch shape as the other element-wise kernels: a workgroup of 256
// threads covers up to 64 16-byte chunk columns of the output (a wave moves
// 1 KiB of a row of each operand) by 256/TW * U rows, one step per workgroup,
// all loads of the step issued first; consecutive workgroups are adjacent
// along a row.
//
// Arithmetic: fp32 throughout, one rounding to the storage type. sigmoid(v) =
// 1 / (1 + e^-v) with the hardware exp2 and reciprocal; erf from the device
// math library.

#include "common.hpp"

#include <cstdlib>

namespace nhp {

constexpr int kGatedThreads = 256;
constexpr int kGatedU = 2;
constexpr int kGatedMaxTw = 64;

enum GateAct {
    kActSwish = NHP_GATE_SWISH,
    kActGelu = NHP_GATE_GELU,
    kActRelu = NHP_GATE_RELU,
    kActSigmoid = NHP_GATE_SIGMOID,
    kActIdentity = NHP_GATE_IDENTITY
};

__device__ __forceinline__ float sigmoid_fast(float v)
{
    return __builtin_amdgcn_rcpf(1.0f + exp2_raw(-v * kLog2e));
}

// act(g) and d act / d g
template <int ACT>
__device__ __forceinline__ void gate_eval(float g, float& act, float& dact)
{
    if constexpr (ACT == kActSwish) {
        const float s = sigmoid_fast(g);
        act = g * s;
        dact = s * (1.0f + g * (1.0f - s));
    } else if constexpr (ACT == kActGelu) {
        const float cdf = 0.5f * (1.0f + erff(g * 0.70710678118654752f));
        const float pdf = 0.3989422804014327f * exp2_raw((-0.5f * kLog2e) * g * g);
        act = g * cdf;
        dact = cdf + g * pdf;
    } else if constexpr (ACT == kActRelu) {
        act = g > 0.0f ? g : 0.0f;
        dact = g > 0.0f ? 1.0f : 0.0f;
    } else if constexpr (ACT == kActSigmoid) {
        const float s = sigmoid_fast(g);
        act = s;
        dact = s * (1.0f - s);
    } else {
        act = g;
        dact = 1.0f;
    }
}

// ---------------------------------------------------------------------------
// BWD = false: out[row, c] = act(g) * x
// BWD = true:  din[row, c] = dy * act(g), din[row, F + c] = dy * x * act'(g)
// `in`: [rows, 2F]; `dy`: [rows, F] (backward only); cprf = chunks per F.
// ---------------------------------------------------------------------------
template <int DT, int ACT, int TW, bool BWD>
__global__ void __launch_bounds__(kGatedThreads)
gated_kernel(void* out, const void* in, const void* dy, const void* bias, uint32_t rows, uint32_t cprf)
{
    constexpr int V = Elt<DT>::kVec;
    constexpr int U = kGatedU;
    constexpr int TR = kGatedThreads / TW;
    using S = typename Elt<DT>::storage;
    const uint32_t tc = threadIdx.x % TW;
    const uint32_t tr = threadIdx.x / TW;
    const uint32_t cc = blockIdx.x * TW + tc;
    if (cc >= cprf) return;
    const size_t f = (size_t)cprf * V;  // features per half
    const size_t col = (size_t)cc * V;
    const S* src = static_cast<const S*>(in);

    float bx[V], bg[V];
#pragma unroll
    for (int j = 0; j < V; ++j) bx[j] = bg[j] = 0.0f;
    if (bias != nullptr) {
        chunk_to_float<DT>(load16(static_cast<const S*>(bias) + col), bx);
        chunk_to_float<DT>(load16(static_cast<const S*>(bias) + f + col), bg);
    }

    const uint32_t r0 = blockIdx.y * (TR * U) + tr;
    u32x4 rx[U], rg[U], rd[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = r0 + u * TR;
        rx[u] = rg[u] = rd[u] = u32x4{0, 0, 0, 0};
        if (row < rows) {
            rx[u] = load16_stream(src + (size_t)row * 2 * f + col);
            rg[u] = load16_stream(src + (size_t)row * 2 * f + f + col);
            if (BWD) rd[u] = load16_stream(static_cast<const S*>(dy) + (size_t)row * f + col);
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = r0 + u * TR;
        if (row < rows) {
            float fx[V], fg[V], fd[V], o0[V], o1[V];
            chunk_to_float<DT>(rx[u], fx);
            chunk_to_float<DT>(rg[u], fg);
            chunk_to_float<DT>(rd[u], fd);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const float x = fx[j] + bx[j];
                const float g = fg[j] + bg[j];
                float act, dact;
                gate_eval<ACT>(g, act, dact);
                if (BWD) {
                    o0[j] = fd[j] * act;
                    o1[j] = (fd[j] * x) * dact;
                } else {
                    o0[j] = act * x;
                }
            }
            if (BWD) {
                S* dst = static_cast<S*>(out) + (size_t)row * 2 * f;
                store16_stream(dst + col, float_to_chunk<DT>(o0));
                store16_stream(dst + f + col, float_to_chunk<DT>(o1));
            } else {
                store16_stream(static_cast<S*>(out) + (size_t)row * f + col, float_to_chunk<DT>(o0));
            }
        }
    }
}

// one thread per output feature, for shapes the chunked layout cannot take
template <int DT, int ACT, bool BWD>
__global__ void __launch_bounds__(kGatedThreads)
gated_scalar_kernel(void* out, const void* in, const void* dy, const void* bias, uint64_t rows, uint64_t f)
{
    const uint64_t i = (uint64_t)blockIdx.x * kGatedThreads + threadIdx.x;
    if (i >= rows * f) return;
    const uint64_t row = i / f, c = i % f;
    float x = Elt<DT>::load(in, (int64_t)(row * 2 * f + c));
    float g = Elt<DT>::load(in, (int64_t)(row * 2 * f + f + c));
    if (bias != nullptr) {
        x = x + Elt<DT>::load(bias, (int64_t)c);
        g = g + Elt<DT>::load(bias, (int64_t)(f + c));
    }
    float act, dact;
    gate_eval<ACT>(g, act, dact);
    if (BWD) {
        const float d = Elt<DT>::load(dy, (int64_t)i);
        Elt<DT>::store(out, (int64_t)(row * 2 * f + c), d * act);
        Elt<DT>::store(out, (int64_t)(row * 2 * f + f + c), (d * x) * dact);
    } else {
        Elt<DT>::store(out, (int64_t)i, act * x);
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
template <int DT, int ACT, bool BWD>
static int gated_launch(void* out, const void* in, const void* dy, const void* bias, int64_t rows, int64_t f,
                        hipStream_t st)
{
    launch_prepare();
    constexpr int V = Elt<DT>::kVec;
    const bool chunked = f % V == 0 && ptr_aligned16(out) && ptr_aligned16(in) && ptr_aligned16(dy) &&
                         ptr_aligned16(bias) && rows < ((int64_t)1 << 31) && f / V < ((int64_t)1 << 31);
    if (chunked) {
        const int64_t cprf = f / V;
        int tw = 1;
        while (tw < kGatedMaxTw && tw < cprf) tw *= 2;
        const int64_t step_rows = (int64_t)(kGatedThreads / tw) * kGatedU;
        const int64_t steps = (rows + step_rows - 1) / step_rows;
        const int64_t col_tiles = (cprf + tw - 1) / tw;
        if (steps <= 65535) {  // grid.y limit; taller tensors take the scalar kernel
            const dim3 grid((uint32_t)col_tiles, (uint32_t)steps);
            if (!grid_fits(col_tiles * steps, kGatedThreads)) return NHP_ERR_SHAPE;
#define CASE(TW_)                                                                                  \
    case TW_:                                                                                      \
        gated_kernel<DT, ACT, TW_, BWD><<<grid, kGatedThreads, 0, st>>>(out, in, dy, bias, (uint32_t)rows, \
                                                                       (uint32_t)cprf);            \
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
    const int64_t total = rows * f;
    const int64_t blocks = (total + kGatedThreads - 1) / kGatedThreads;
    if (!grid_fits(blocks, kGatedThreads)) return NHP_ERR_SHAPE;
    gated_scalar_kernel<DT, ACT, BWD><<<(uint32_t)blocks, kGatedThreads, 0, st>>>(out, in, dy, bias, (uint64_t)rows,
                                                                                (uint64_t)f);
    return launch_result();
}

template <int DT, bool BWD>
static int gated_by_act(void* out, const void* in, const void* dy, const void* bias, int64_t rows, int64_t f, int act,
                        hipStream_t st)
{
    switch (act) {
    case kActSwish:
        return gated_launch<DT, kActSwish, BWD>(out, in, dy, bias, rows, f, st);
    case kActGelu:
        return gated_launch<DT, kActGelu, BWD>(out, in, dy, bias, rows, f, st);
    case kActRelu:
        return gated_launch<DT, kActRelu, BWD>(out, in, dy, bias, rows, f, st);
    case kActSigmoid:
        return gated_launch<DT, kActSigmoid, BWD>(out, in, dy, bias, rows, f, st);
    case kActIdentity:
        return gated_launch<DT, kActIdentity, BWD>(out, in, dy, bias, rows, f, st);
    default:
        return NHP_ERR_SHAPE;
    }
}

template <bool BWD>
static int gated_entry(void* out, const void* in, const void* dy, const void* bias, int64_t rows, int64_t f, int act,
                       int dtype, void* stream)
{
    if (dtype != NHP_F16 && dtype != NHP_BF16 && dtype != NHP_F32) return NHP_ERR_DTYPE;
    if (act < kActSwish || act > kActIdentity) return NHP_ERR_SHAPE;
    if (rows < 0 || f < 0) return NHP_ERR_SHAPE;
    if (rows > 0 && f > ((int64_t)1 << 61) / rows) return NHP_ERR_SHAPE;
    if (rows == 0 || f == 0) return NHP_OK;
    if (!out || !in || (BWD && !dy)) return NHP_ERR_NULL;
    if (out == in) return NHP_ERR_ALIAS;  // the two halves of a row are read by other threads than write them
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case NHP_F16:
        return gated_by_act<NHP_F16, BWD>(out, in, dy, bias, rows, f, act, st);
    case NHP_BF16:
        return gated_by_act<NHP_BF16, BWD>(out, in, dy, bias, rows, f, act, st);
    default:
        return gated_by_act<NHP_F32, BWD>(out, in, dy, bias, rows, f, act, st);
    }
}

}  // namespace nhp

using namespace nhp;

extern "C" {

int nhp_gated_act_fwd(void* out, const void* in, const void* bias, int64_t rows, int64_t features, int act,
                      int dtype, void* stream)
{
    return gated_entry<false>(out, in, nullptr, bias, rows, features, act, dtype, stream);
}

int nhp_gated_act_bwd(void* din, const void* dy, const void* in, const void* bias, int64_t rows, int64_t features,
                      int act, int dtype, void* stream)
{
    return gated_entry<true>(din, in, dy, bias, rows, features, act, dtype, stream);
}

}  // extern "C"
