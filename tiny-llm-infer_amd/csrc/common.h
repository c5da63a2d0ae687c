// Shared by all kernels: storage types, conversions, reductions over a
// 64-lane wavefront and over a workgroup, and the error channel of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TLI_WAVE 64

typedef uint16_t bf16_t;   // bfloat16 storage: the upper 16 bits of a float

// dtype codes of the C ABI
#define TLI_F32 0
#define TLI_BF16 1

// The chip that the launch rules deal work out to.  Workgroups go round the dies in turn, and
// every die has an L2 cache of its own.  The runtime reports the compute units of a device but
// not its dies, so their number is the one constant: 8 on MI355X, of 32 compute units each.
#define TLI_DIES 8
int tli_compute_units();                     // of the current device, asked once (256 on MI355X)
static inline int tli_units_a_die() { return tli_compute_units() / TLI_DIES; }

extern "C" const char* tli_last_error();
int tli_fail(const char* fmt, ...);          // records a message, returns 1
int tli_check_launch(const char* what);      // hipGetLastError -> message

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest, ties to even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    const __bf16 b = (__bf16)f;
    return *reinterpret_cast<const bf16_t*>(&b);
}

// two at once: low half = a, high half = b
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    const bf16x2_t r = __builtin_convertvector((f32x2_t){a, b}, bf16x2_t);
    return *reinterpret_cast<const uint32_t*>(&r);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ void from_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void from_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// A value on its way into the cache: infinities and NaNs become 0.  The MFMA attention
// kernels multiply values of keys that a row does not see by a weight of exactly 0, which
// only gives 0 for finite values; a page is used again by other requests.
__device__ __forceinline__ bf16_t cache_value(bf16_t v) { return (v & 0x7F80u) == 0x7F80u ? (bf16_t)0 : v; }
__device__ __forceinline__ float cache_value(float v) { return (__float_as_uint(v) & 0x7F800000u) == 0x7F800000u ? 0.f : v; }

// Four values that a lane holds for four consecutive columns, as one store where the row allows it
// (`left`: columns from dst to the row's end; `whole`: every row starts a multiple of four columns
// in, so that the store is aligned), else one by one.
__device__ __forceinline__ void store4(float* dst, const float (&v)[4], int left, bool whole) {
    if (left >= 4 && whole) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (i < left) dst[i] = v[i];
}
__device__ __forceinline__ void store4(bf16_t* dst, const float (&v)[4], int left, bool whole) {
    if (left >= 4 && whole) {
        *reinterpret_cast<uint2*>(dst) = make_uint2((uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16),
                                                    (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16));
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (i < left) dst[i] = f32_to_bf16(v[i]);
}

// Makes LDS writes of this wavefront's lanes visible to its other lanes.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Maximum / sum over the four lanes l, l^16, l^32, l^48 (the lane groups of an MFMA
// tile), every lane gets the result.  v_permlane16_swap / v_permlane32_swap exchange
// rows of 16 (halves of 32) lanes between two registers without going through LDS:
// with both operands holding x, one result has the even rows (lower half) twice and the
// other the odd rows (upper half) twice, so combining the two is the exchange with l^16
// (l^32) done for every lane at once.
__device__ __forceinline__ float quad_rows_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float m = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const uint32_t v = __float_as_uint(m);
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ float quad_rows_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float m = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const uint32_t v = __float_as_uint(m);
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// One element of a rotated pair.  The roundings are written out (a product rounded, then one fused
// multiply-add) so that every kernel that rotates gives the same bits: left to the compiler, which of the
// two products of `a b + c d` is fused depends on the code around it.
// first half of a head: x cos - partner sin;  second half: partner sin + x cos
__device__ __forceinline__ float rotate_first_half(float x, float partner, float cs, float sn) {
    return fmaf(x, cs, -(partner * sn));
}
__device__ __forceinline__ float rotate_second_half(float x, float partner, float cs, float sn) {
    return fmaf(partner, sn, x * cs);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = TLI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TLI_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = TLI_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TLI_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS.  The order of additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    const int waves = (blockDim.x + TLI_WAVE - 1) / TLI_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    const int waves = (blockDim.x + TLI_WAVE - 1) / TLI_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
    return total;
}
