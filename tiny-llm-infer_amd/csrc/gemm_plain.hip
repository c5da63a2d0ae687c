// Plain tiled matrix product y[M,N] = x[M,K] . W[N,K]^T for any sizes and for
// float32 or bfloat16 inputs, float32 accumulation in a fixed order (k
// ascending, no split over k), so a row's result does not depend on how many
// other rows are in the batch.  This is the matrix product of the float32 path
// (plain FMA, no reduced-precision matrix mode) and the reference beside the
// MFMA kernels.  Weights are [out, in] row-major as the reference stores them
// (kernels/src/matmul_kernel_cpu.cpp:27-35).
#include "common.h"

#define GP_TILE 64
#define GP_K 16

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const TX* __restrict__ x, const TW* __restrict__ w, TY* __restrict__ y,
                  int M, int N, int K) {
    __shared__ float xs[GP_K][GP_TILE + 1];
    __shared__ float ws[GP_K][GP_TILE + 1];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int m0 = blockIdx.y * GP_TILE, n0 = blockIdx.x * GP_TILE;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GP_K) {
        // 64 rows x 16 k of each operand: 1024 elements, 4 per thread
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = threadIdx.x + e * 256;
            const int r = idx / GP_K, kk = idx % GP_K;
            const int k = k0 + kk;
            xs[kk][r] = (m0 + r < M && k < K) ? to_f32(x[(size_t)(m0 + r) * K + k]) : 0.f;
            ws[kk][r] = (n0 + r < N && k < K) ? to_f32(w[(size_t)(n0 + r) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GP_K; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) from_f32(y + (size_t)m * N + n, acc[i][j]);
        }
    }
}

// dtype codes: x_dtype/w_dtype/y_dtype in {TLI_F32, TLI_BF16}
extern "C" int tli_gemm_plain(const void* x, const void* w, void* y, int M, int N, int K,
                              int x_dtype, int w_dtype, int y_dtype, void* stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return tli_fail("gemm: K must be positive, got %d", K);
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((N + GP_TILE - 1) / GP_TILE, (M + GP_TILE - 1) / GP_TILE);
    if (grid.y > 65535) return tli_fail("gemm: %d rows exceed the grid limit", M);
    if (x_dtype == TLI_F32 && w_dtype == TLI_F32 && y_dtype == TLI_F32)
        gemm_plain_kernel<float, float, float><<<grid, 256, 0, s>>>(
            (const float*)x, (const float*)w, (float*)y, M, N, K);
    else if (x_dtype == TLI_BF16 && w_dtype == TLI_BF16 && y_dtype == TLI_BF16)
        gemm_plain_kernel<bf16_t, bf16_t, bf16_t><<<grid, 256, 0, s>>>(
            (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, M, N, K);
    else if (x_dtype == TLI_BF16 && w_dtype == TLI_BF16 && y_dtype == TLI_F32)
        gemm_plain_kernel<bf16_t, bf16_t, float><<<grid, 256, 0, s>>>(
            (const bf16_t*)x, (const bf16_t*)w, (float*)y, M, N, K);
    else
        return tli_fail("gemm: unsupported dtype combination x=%d w=%d y=%d", x_dtype, w_dtype, y_dtype);
    return tli_check_launch("gemm_plain");
}
