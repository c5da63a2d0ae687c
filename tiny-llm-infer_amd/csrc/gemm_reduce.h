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

// The same for four consecutive output columns a thread (N a multiple of 4; of 32 if gated): one
// 16-byte load a plane and one store.
template <typename TO>
__global__ void gemm_mid_reduce4_kernel(const float* __restrict__ part, TO* __restrict__ y, int M, int N,
                                        int splits, int gated) {
    const int n_out = gated ? N / 2 : N, quads = n_out / 4;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * quads) return;
    const int row = (int)(idx / quads), j = (int)(idx % quads) * 4;
    const size_t plane = (size_t)M * N;
    float o[4];
    if (gated) {
        const size_t gcol = (size_t)(j / 16) * 32 + j % 16;
        float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < splits; ++s) {
            const float4 a = *reinterpret_cast<const float4*>(part + s * plane + (size_t)row * N + gcol);
            const float4 b = *reinterpret_cast<const float4*>(part + s * plane + (size_t)row * N + gcol + 16);
            g[0] += a.x; g[1] += a.y; g[2] += a.z; g[3] += a.w;
            u[0] += b.x; u[1] += b.y; u[2] += b.z; u[3] += b.w;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = g[i] / (1.0f + expf(-g[i])) * u[i];
    } else {
        o[0] = o[1] = o[2] = o[3] = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float4 a = *reinterpret_cast<const float4*>(part + s * plane + (size_t)row * N + j);
            o[0] += a.x; o[1] += a.y; o[2] += a.z; o[3] += a.w;
        }
    }
    store4(y + (size_t)row * n_out + j, o, 4, true);
}

// Launches the pass: four columns a thread where the sizes and addresses allow it.
template <typename TO>
static inline void launch_gemm_reduce(const float* part, TO* y, int M, int N, int splits, int gated, hipStream_t s) {
    const int n_out = gated ? N / 2 : N;
    if (N % 4 == 0 && n_out % 4 == 0 && !(((uintptr_t)part | (uintptr_t)y) & 15)) {
        const size_t total = (size_t)M * (n_out / 4);
        gemm_mid_reduce4_kernel<TO><<<(unsigned)((total + 255) / 256), 256, 0, s>>>(part, y, M, N, splits, gated);
    } else {
        const size_t total = (size_t)M * n_out;
        gemm_mid_reduce_kernel<TO><<<(unsigned)((total + 255) / 256), 256, 0, s>>>(part, y, M, N, splits, gated);
    }
}
