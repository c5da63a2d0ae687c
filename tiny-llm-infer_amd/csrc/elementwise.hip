// Embedding gather, residual-add + RMSNorm, SwiGLU.
//
// embed:       resid[t, :] = float(table[id[t], :])                       (layers/src/embedding.cpp:37-44)
// add_rmsnorm: v = resid[r] (+ delta[r]);  out = w * v * 1/sqrt(mean(v^2) + eps), in float32
//              (kernels/src/rmsnorm_kernel_cpu.cpp:27-43; the sum h + a of
//              model/src/qwen3_paged_batch.cpp:273-275 is done here, unrounded).
//              delta may also come as float32 partial sums [parts][rows][n] of a matrix
//              product whose k range was split: they are added in order and rounded to
//              bfloat16 first, which is what the product's own reduction would have stored
// swiglu:      out = g / (1 + exp(-g)) * u over a fused [rows, 2*inter] input
//              (kernels/src/swiglu_kernel_cpu.cpp:20-24)
#include "common.h"

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int hidden, int vocab) {
    const int row = blockIdx.x;
    int id = ids[row];
    if (id < 0 || id >= vocab) id = 0;          // the host rejects such ids before the launch
    const T* src = table + (size_t)id * hidden;
    float* dst = out + (size_t)row * hidden;
    if (sizeof(T) == 2 && hidden % 8 == 0 && !(((uintptr_t)table | (uintptr_t)out) & 15)) {
        // eight elements a thread and turn: one 16-byte load, two 16-byte stores
        for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
            const uint4 v = *reinterpret_cast<const uint4*>(src + i);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            float f[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f[2 * e] = __uint_as_float(w[e] << 16);
                f[2 * e + 1] = __uint_as_float(w[e] & 0xFFFF0000u);
            }
            *reinterpret_cast<float4*>(dst + i) = make_float4(f[0], f[1], f[2], f[3]);
            *reinterpret_cast<float4*>(dst + i + 4) = make_float4(f[4], f[5], f[6], f[7]);
        }
        return;
    }
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32(src[i]);
}

// What a row owes the residual: a row of T, or float32 partial sums [parts][total_rows][n]
// added in order and rounded to bfloat16.
template <typename T>
struct RowDelta {
    const T* d;
    const float* p;
    int parts;
    size_t plane;
    __device__ __forceinline__ bool any() const { return d != nullptr || parts > 0; }
    __device__ __forceinline__ float at(int i) const {
        if (parts > 0) {
            float a = 0.f;
            for (int s = 0; s < parts; ++s) a += p[s * plane + i];
            return bf16_to_f32(f32_to_bf16(a));
        }
        return to_f32(d[i]);
    }
};

template <typename T>
__device__ __forceinline__ RowDelta<T> row_delta(const void* delta, int parts, int r, int n, int total_rows) {
    RowDelta<T> rd{nullptr, nullptr, parts, (size_t)total_rows * n};
    if (parts > 0) rd.p = (const float*)delta + (size_t)r * n;
    else if (delta) rd.d = (const T*)delta + (size_t)r * n;
    return rd;
}

template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const void* __restrict__ delta, int parts,
                                   const float* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int n, float eps, int total_rows) {
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    int r = rows ? rows[out_row] : out_row;
    if (r < 0 || r >= total_rows) r = 0;
    float* x = resid + (size_t)r * n;
    const RowDelta<T> d = row_delta<T>(delta, parts, r, n, total_rows);
    const bool update = (rows == nullptr) && d.any();
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = x[i];
        if (d.any()) v += d.at(i);
        if (update) x[i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    T* o = out + (size_t)out_row * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = x[i];
        if (d.any() && !update) v += d.at(i);
        from_f32(o + i, weight[i] * v * scale);
    }
}

// The same with the row held in registers: n % 4 == 0 and n <= 4 * blockDim.x * IT.
// Each thread owns IT groups of 4 consecutive elements, read and written once.
__device__ __forceinline__ void load4(const float* p, float v[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float v[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = bf16_to_f32((bf16_t)(t.x & 0xffffu)); v[1] = bf16_to_f32((bf16_t)(t.x >> 16));
    v[2] = bf16_to_f32((bf16_t)(t.y & 0xffffu)); v[3] = bf16_to_f32((bf16_t)(t.y >> 16));
}
__device__ __forceinline__ void store4(float* p, const float v[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float v[4]) {
    uint2 t;
    t.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
    t.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

template <typename T, int IT>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ resid, const void* __restrict__ delta, int parts,
                                       const float* __restrict__ weight, T* __restrict__ out,
                                       const int* __restrict__ rows, int n, float eps, int total_rows) {
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    int r = rows ? rows[out_row] : out_row;
    if (r < 0 || r >= total_rows) r = 0;
    float* x = resid + (size_t)r * n;
    const RowDelta<T> d = row_delta<T>(delta, parts, r, n, total_rows);
    const bool update = (rows == nullptr) && d.any();
    float v[IT][4], w[IT][4];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (threadIdx.x + it * blockDim.x) * 4;
        if (i < n) {
            load4(x + i, v[it]);
            load4(weight + i, w[it]);         // asked for now: after the sum it would be one more wait for memory
            if (d.any()) {
                float dv[4];
                if (d.parts > 0) {
                    // four planes a round, all asked for before any is added (in plane order; a plane
                    // past the last is the last again and is not added)
                    float a[4] = {0.f, 0.f, 0.f, 0.f};
                    for (int s = 0; s < d.parts; s += 4) {
                        float pv[4][4];
#pragma unroll
                        for (int k = 0; k < 4; ++k) load4(d.p + (size_t)min(s + k, d.parts - 1) * d.plane + i, pv[k]);
#pragma unroll
                        for (int k = 0; k < 4; ++k)
#pragma unroll
                            for (int e = 0; e < 4; ++e) a[e] = s + k < d.parts ? a[e] + pv[k][e] : a[e];
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) dv[e] = bf16_to_f32(f32_to_bf16(a[e]));
                } else {
                    load4(d.d + i, dv);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) v[it][e] += dv[e];
                if (update) store4(x + i, v[it]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) ss += v[it][e] * v[it][e];
        }
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    T* o = out + (size_t)out_row * n;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (threadIdx.x + it * blockDim.x) * 4;
        if (i < n) {
            float y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = w[it][e] * v[it][e] * scale;
            store4(o + i, y);
        }
    }
}

template <typename T>
static void launch_add_rmsnorm(float* resid, const void* delta, int parts, const float* weight, T* out,
                               const int* rows, int out_rows, int total_rows, int n, float eps, hipStream_t s) {
    const int groups = n / 4;
    if (n % 4 == 0 && groups <= 4096) {
        int threads = groups <= 1024 ? (groups + 63) / 64 * 64 : 1024;
        if (groups <= 1024)
            add_rmsnorm_vec_kernel<T, 1><<<out_rows, threads, 0, s>>>(resid, delta, parts, weight, out, rows, n, eps, total_rows);
        else if (groups <= 2048)
            add_rmsnorm_vec_kernel<T, 2><<<out_rows, threads, 0, s>>>(resid, delta, parts, weight, out, rows, n, eps, total_rows);
        else
            add_rmsnorm_vec_kernel<T, 4><<<out_rows, threads, 0, s>>>(resid, delta, parts, weight, out, rows, n, eps, total_rows);
        return;
    }
    add_rmsnorm_kernel<T><<<out_rows, n >= 2048 ? 512 : 256, 0, s>>>(resid, delta, parts, weight, out, rows, n, eps, total_rows);
}

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t row = idx / inter;
    const int col = (int)(idx - row * inter);
    const float g = to_f32(gu[row * 2 * inter + col]);
    const float u = to_f32(gu[row * 2 * inter + inter + col]);
    from_f32(out + idx, g / (1.0f + expf(-g)) * u);
}

// token_ids[r] = src[from[r]] where from[r] >= 0: the tokens a step sampled become the
// next step's inputs without leaving the device
__global__ void feed_tokens_kernel(int* __restrict__ token_ids, const int* __restrict__ from,
                                   const int* __restrict__ src, int rows, int src_count) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const int f = from[r];
    if (f >= 0 && f < src_count) token_ids[r] = src[f];
}

extern "C" int tli_feed_tokens(int* token_ids, const int* from, const int* src, int rows, int src_count,
                               void* stream) {
    if (rows <= 0) return 0;
    feed_tokens_kernel<<<(rows + 255) / 256, 256, 0, (hipStream_t)stream>>>(token_ids, from, src, rows, src_count);
    return tli_check_launch("feed_tokens");
}

extern "C" int tli_embed(const void* table, const int* ids, float* out, int rows, int hidden,
                         int vocab, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (hidden <= 0 || vocab <= 0) return tli_fail("embed: bad sizes hidden=%d vocab=%d", hidden, vocab);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        embed_kernel<float><<<rows, 256, 0, s>>>((const float*)table, ids, out, hidden, vocab);
    else if (dtype == TLI_BF16)
        embed_kernel<bf16_t><<<rows, 256, 0, s>>>((const bf16_t*)table, ids, out, hidden, vocab);
    else
        return tli_fail("embed: unknown dtype %d", dtype);
    return tli_check_launch("embed");
}

// parts > 0: `delta` holds float32 partial sums [parts][total_rows][n] (bfloat16 rows only).
extern "C" int tli_add_rmsnorm(float* resid, const void* delta, const float* weight, void* out,
                               const int* rows, int out_rows, int total_rows, int n, float eps,
                               int dtype, int parts, void* stream) {
    if (out_rows <= 0) return 0;
    if (n <= 0) return tli_fail("add_rmsnorm: bad row size %d", n);
    if (parts < 0 || (parts > 0 && (dtype != TLI_BF16 || !delta)))
        return tli_fail("add_rmsnorm: partial sums (%d) go with bfloat16 rows only", parts);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        launch_add_rmsnorm<float>(resid, delta, 0, weight, (float*)out, rows, out_rows, total_rows, n, eps, s);
    else if (dtype == TLI_BF16)
        launch_add_rmsnorm<bf16_t>(resid, delta, parts, weight, (bf16_t*)out, rows, out_rows, total_rows, n,
                                   eps, s);
    else
        return tli_fail("add_rmsnorm: unknown dtype %d", dtype);
    return tli_check_launch("add_rmsnorm");
}

// 8 outputs a thread, 16-byte loads: inter % 8 == 0
__global__ void swiglu_vec_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int inter,
                                  size_t groups) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= groups) return;
    const int per_row = inter / 8;
    const size_t row = idx / per_row;
    const int col = (int)(idx - row * per_row) * 8;
    const uint4 g4 = *reinterpret_cast<const uint4*>(gu + row * 2 * inter + col);
    const uint4 u4 = *reinterpret_cast<const uint4*>(gu + row * 2 * inter + inter + col);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float g0 = bf16_to_f32((bf16_t)(gw[i] & 0xffffu)), g1 = bf16_to_f32((bf16_t)(gw[i] >> 16));
        const float u0 = bf16_to_f32((bf16_t)(uw[i] & 0xffffu)), u1 = bf16_to_f32((bf16_t)(uw[i] >> 16));
        const float a0 = g0 / (1.0f + expf(-g0)) * u0, a1 = g1 / (1.0f + expf(-g1)) * u1;
        ow[i] = (uint32_t)f32_to_bf16(a0) | ((uint32_t)f32_to_bf16(a1) << 16);
    }
    *reinterpret_cast<uint4*>(out + row * inter + col) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int tli_swiglu(const void* gu, void* out, int rows, int inter, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (inter <= 0) return tli_fail("swiglu: bad size %d", inter);
    hipStream_t s = (hipStream_t)stream;
    const size_t total = (size_t)rows * inter;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (dtype == TLI_F32)
        swiglu_kernel<float><<<blocks, 256, 0, s>>>((const float*)gu, (float*)out, inter, total);
    else if (dtype == TLI_BF16 && inter % 8 == 0) {
        const size_t groups = total / 8;
        swiglu_vec_kernel<<<(unsigned)((groups + 255) / 256), 256, 0, s>>>((const bf16_t*)gu, (bf16_t*)out, inter, groups);
    } else if (dtype == TLI_BF16)
        swiglu_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)gu, (bf16_t*)out, inter, total);
    else
        return tli_fail("swiglu: unknown dtype %d", dtype);
    return tli_check_launch("swiglu");
}
