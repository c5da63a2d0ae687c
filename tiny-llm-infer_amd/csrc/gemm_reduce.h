// The pass that adds the float32 partial products of a matrix product whose k range was
// split over workgroups (gemm_mid.hip, gemm_rows.hip), in split order.
#pragma once
#include "common.h"

// Sum of the partial products in split order.  gated: output column j of [M, N/2] takes
// gate column (j/16)*32 + j%16 and up column 16 further.
template <typename TO>
__global__ void gemm_mid_reduce_kernel(const float* __restrict__ part, TO* __restrict__ y, int M, int N,
                                       int splits, int gated) {
    const int n_out = gated ? N / 2 : N;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * n_out) return;
    const int row = (int)(idx / n_out), j = (int)(idx % n_out);
    const size_t plane = (size_t)M * N;
    if (gated) {
        const size_t gcol = (size_t)(j / 16) * 32 + j % 16;
        float g = 0.f, u = 0.f;
        for (int s = 0; s < splits; ++s) {
            g += part[s * plane + (size_t)row * N + gcol];
            u += part[s * plane + (size_t)row * N + gcol + 16];
        }
        from_f32(y + idx, g / (1.0f + expf(-g)) * u);
    } else {
        float v = 0.f;
        for (int s = 0; s < splits; ++s) v += part[s * plane + (size_t)row * N + j];
        from_f32(y + idx, v);
    }
}
