// Second stage of the column reductions: adds up the fp32 partial rows that the
// workgroups of a first-stage kernel wrote, in a fixed order.
#pragma once

#include "common.hpp"

namespace nhp {

// out[c] = sum over t of partial[t][c], stored as fp32 or as DT. A workgroup of 1024 threads
// takes 32 columns by 32 slices of t (a thread adds the rows t = slice, slice + 32, ...,
// eight loads in flight), then the slices are added in a fixed order through LDS.
// blockIdx.y selects the (partial, out) pair.
constexpr int kFinishCols = 32, kFinishSlices = 32;

template <int DT>
__global__ void __launch_bounds__(kFinishCols* kFinishSlices)
partial_rows_sum_kernel(void* out0, void* out1, const float* part0, const float* part1, uint32_t tiles,
                         uint32_t cols, int out_f32)
{
    __shared__ float lds[kFinishSlices][kFinishCols + 1];
    void* out = blockIdx.y == 0 ? out0 : out1;
    const float* partial = blockIdx.y == 0 ? part0 : part1;
    if (out == nullptr) return;
    const uint32_t tx = threadIdx.x % kFinishCols, ty = threadIdx.x / kFinishCols;
    const uint32_t c = blockIdx.x * kFinishCols + tx;
    float s = 0.0f;
    if (c < cols) {
        uint32_t t = ty;
        for (; t + 7 * kFinishSlices < tiles; t += 8 * kFinishSlices) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = partial[(size_t)(t + i * kFinishSlices) * cols + c];
#pragma unroll
            for (int i = 0; i < 8; ++i) s += v[i];
        }
        for (; t < tiles; t += kFinishSlices) s += partial[(size_t)t * cols + c];
    }
    lds[ty][tx] = s;
    __syncthreads();
    if (ty == 0 && c < cols) {
        float r = lds[0][tx];
#pragma unroll
        for (int i = 1; i < kFinishSlices; ++i) r += lds[i][tx];
        if (out_f32)
            static_cast<float*>(out)[c] = r;
        else
            Elt<DT>::store(out, c, r);
    }
}

}  // namespace nhp
