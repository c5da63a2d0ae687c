// Matrix product for few rows (decode): y[M,N] = x[M,K] . W[N,K]^T, M <= 64,
// bfloat16 inputs, float32 accumulation on the matrix cores, bfloat16 or
// float32 output.  The work is streaming W from HBM once; everything is laid
// out so that each lane's global loads are 64 contiguous bytes of one W row and
// land directly in the MFMA operand registers (no LDS staging of W).
//
// The reference multiplies a single row with a hand GEMV and more rows with a
// library call (kernels/src/matmul_kernel_cuda.cu:72-91); this kernel covers
// both for up to 64 rows.
//
// v_mfma_f32_16x16x32_bf16 computes D[16x16] += A[16x32] B[32x16]; lane l holds
// A[l%16][(l/16)*8 .. +8], B[(l/16)*8 .. +8][l%16] and D[(l/16)*4 .. +4][l%16].
// Here A is a tile of W (16 output columns n), B is x^T (16 rows m), so a lane
// ends with y[m = l%16][n = (l/16)*4 .. +4].  The 32 k-slots of one MFMA may be
// any 32 values of k as long as A and B agree: lane group c = l/16 takes the 32
// consecutive k  [kb + 32c, kb + 32c + 32)  of a 128-wide step, 8 per MFMA.
//
// A workgroup owns 16*RT output columns; its waves take the 128-wide k steps in
// turn and their partial sums are added through LDS in wave order, so the
// result does not depend on the launch.
//
// Two variants take the RMS norms of a decoder block into the products around them, so
// that a decode step needs no norm kernel between its products.  With h the float32
// residual, w the norm's weights and r = 1/sqrt(mean(h^2) + eps) of a row, the normed row
// is w*h*r, and (w*h*r) . W^T = r * ((w*h) . W^T): the scalar r can wait until after the
// product.
//   FUSE_RESIDUAL (output projections): h += x . W^T in float32, then the product writes
//       bfloat16(w*h) for the next product and, for every 16 columns, the rows' partial
//       sums of h^2.
//   FUSE_RSTD (the products that read normed rows): x is such a bfloat16(w*h); the rows'
//       partial sums are added in order, and the outputs are scaled by r (before the
//       SwiGLU of a gated matrix).
// Sums, r and the residual are float32 (kernels/src/rmsnorm_kernel_cpu.cpp:27-43); the
// rounding to bfloat16 happens once, as for a separate norm, only before r is applied
// instead of after (a scalar factor does not change the relative rounding error).
#include "common.h"
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
union Pack16 {
    uint4 u;
    u32x4_t w;
    bf16x8 v;
};

// 16 bytes of a matrix that a step reads once, in the tiled layout (a load instruction of a
// wave takes 1 KiB in a row): a non-temporal load, so that the caches do not keep 16 GB of
// weights a step in place of the little that every kernel begins with (activations, norm
// weights, positions, block tables).  Measured at the Qwen3-8B shape: 3.37 -> 3.13 ms a step at
// batch 8, 13.8k -> 14.5k tokens/s at batch 64.  Not for loads that take a line in pieces:
// the key fragments of the decode attention as non-temporal loads made its step 3% slower.
__device__ __forceinline__ u32x4_t load16_once(const bf16_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
}

__device__ __forceinline__ uint4 load16_or_zero(const bf16_t* p, bool ok) {
    return ok ? *reinterpret_cast<const uint4*>(p) : make_uint4(0, 0, 0, 0);
}

#define FUSE_NONE 0
#define FUSE_RSTD 1
#define FUSE_RESIDUAL 2

struct SkinnyFuse {
    const float* ssq_in;      // FUSE_RSTD: [parts_in][M] partial sums of squares of the rows of x's source
    int parts_in;
    float eps;
    float* resid;             // FUSE_RESIDUAL: [M][N] float32, updated in place
    const float* norm_w;      // [N] weights of the norm that follows
    bf16_t* xw;               // [M][N] bfloat16(norm_w * resid)
    float* ssq_out;           // [ceil(N/16)][M]
};

template <int RT, int MT, int WAVES, typename TO, bool TILED = false, bool GATED = false, int DEPTH = 2,
          int FUSE = FUSE_NONE>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, TO* __restrict__ y,
                   int M, int N, int K, SkinnyFuse fuse) {
    __shared__ float red[WAVES][RT * MT][64][4];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int r = lane % 16, c = lane / 16;
    const int n_base = blockIdx.x * (16 * RT);

    f32x4 acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // Rows past the end read a valid row instead (w: row 0, x: the last row) and are
    // never stored, so that no load of the main loop is predicated.
    const bf16_t* w_row[RT];
    bool w_ok[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int n = n_base + t * 16 + r;
        w_ok[t] = n < N;
        w_row[t] = w + (size_t)(w_ok[t] ? n : 0) * K;
        if (TILED)   // blocks of 16 rows x 128 k = 4 KiB, stored [j][lane][8]: one load instruction
                     // of a wave reads 1 KiB in a row
            w_row[t] = w + ((size_t)(blockIdx.x * RT + t) * ((K + 127) / 128)) * 2048 + lane * 8;
    }
    const bf16_t* x_row[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) x_row[m] = x + (size_t)min(m * 16 + r, M - 1) * K;

    // Ring of DEPTH register stages: the loads of the next DEPTH-1 128-wide steps are in
    // flight while the MFMAs of the current one run, so a wave keeps up to
    // 4*(RT+MT)*(DEPTH-1) 16-byte loads in flight.  The main loop takes whole steps only
    // and none of its loads is under a branch: after a branch that may have issued loads
    // the compiler waits for all loads in flight, which would undo the prefetching.
    Pack16 a[DEPTH][RT][4], b[DEPTH][MT][4];
    auto load_step = [&](auto STAGE, int kb) {
        constexpr int S = decltype(STAGE)::value;
        const int k = kb + c * 32;
        // x first: it comes from L2 and loads complete in the order of issue
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                b[S][m][j].u = *reinterpret_cast<const uint4*>(x_row[m] + k + j * 8);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < RT; ++t)
                if (TILED)
                    a[S][t][j].w = load16_once(w_row[t] + (size_t)(kb / 128) * 2048 + j * 512);
                else
                    a[S][t][j].u = *reinterpret_cast<const uint4*>(w_row[t] + k + j * 8);
    };
    auto mma_step = [&](auto STAGE) {
        constexpr int S = decltype(STAGE)::value;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[S][t][j].v, b[S][m][j].v,
                                                                        acc[t][m], 0, 0, 0);
        // keeps the scheduler from moving the loads of the next step (issued after this
        // in program order) ahead of these products, where they would have to be waited
        // for together with the operands used here
        __builtin_amdgcn_sched_barrier(0);
    };
    // this wave's whole steps: number i is at k = (wave + i*WAVES) * 128
    const int whole = K / 128;
    const int mine = wave < whole ? (whole - wave + WAVES - 1) / WAVES : 0;
    auto k_of = [&](int i) { return (wave + i * WAVES) * 128; };
    auto prologue = [&](auto self, auto INDEX) -> void {
        constexpr int I = decltype(INDEX)::value;
        if constexpr (I < DEPTH - 1) {
            if (I < mine) load_step(std::integral_constant<int, I>{}, k_of(I));
            self(self, std::integral_constant<int, I + 1>{});
        }
    };
    // a round: step i + I multiplies stage I after the load of step i + I + DEPTH - 1 went out
    auto round = [&](auto self, int i, auto INDEX, auto FULL_T) -> void {
        constexpr int I = decltype(INDEX)::value;
        constexpr bool FULL = decltype(FULL_T)::value;
        if constexpr (I < DEPTH) {
            if (FULL || i + I < mine) {
                if (FULL || i + I + DEPTH - 1 < mine)
                    load_step(std::integral_constant<int, (I + DEPTH - 1) % DEPTH>{}, k_of(i + I + DEPTH - 1));
                __builtin_amdgcn_sched_barrier(0);
                mma_step(std::integral_constant<int, I>{});
                self(self, i, std::integral_constant<int, I + 1>{}, FULL_T);
            }
        }
    };
    prologue(prologue, std::integral_constant<int, 0>{});
    // (asked for behind the first W fragments, needed only after the last)
    // FUSE_RSTD: the partial sums of squares are shared out over the waves and lane groups
    // (part p to wave (p / 4) % WAVES, lane group p % 4), asked for eight at a time without
    // a branch, and added up over the workgroup only after the main loop
    float ssq_mine[MT];
    if (FUSE == FUSE_RSTD) {
        constexpr int STEP = 4 * WAVES;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = min(m * 16 + r, M - 1);
            float a = 0.f;
            for (int p0 = wave * 4 + c; p0 < fuse.parts_in; p0 += 8 * STEP) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int p = p0 + e * STEP;
                    v[e] = fuse.ssq_in[(size_t)min(p, fuse.parts_in - 1) * M + row] * (p < fuse.parts_in ? 1.f : 0.f);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) a += v[e];
            }
            ssq_mine[m] = quad_rows_sum(a);            // over the four lane groups
        }
    }
    float h_old[4] = {0.f, 0.f, 0.f, 0.f}, nw[4] = {0.f, 0.f, 0.f, 0.f};
    if (FUSE == FUSE_RESIDUAL) {
        static_assert(FUSE != FUSE_RESIDUAL || (MT == 1 && RT <= WAVES), "one tile a wave at most");
        {   // wave t < RT finishes tile t: its residual values and norm weights (the other
            // waves ask for the same as wave 0, which costs nothing and keeps the loads
            // free of branches; rows and columns past the end repeat the last)
            const int n0 = n_base + (wave < RT ? wave : 0) * 16 + c * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = min(n0 + e, N - 1);
                h_old[e] = fuse.resid[(size_t)min(r, M - 1) * N + col];
                nw[e] = fuse.norm_w[col];
            }
        }
    }
    int i = 0;
    for (; i + 2 * (DEPTH - 1) < mine; i += DEPTH)
        round(round, i, std::integral_constant<int, 0>{}, std::true_type{});
    for (; i < mine; i += DEPTH)
        round(round, i, std::integral_constant<int, 0>{}, std::false_type{});
    // the last, partial step of k belongs to the wave whose turn it is; it comes after
    // that wave's whole steps, as it would in one loop over all steps
    if (K % 128 && wave == whole % WAVES) {
        const int k = whole * 128 + c * 32;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool in = k + j * 8 < K;
#pragma unroll
            for (int t = 0; t < RT; ++t)
                a[0][t][j].u = TILED ? *reinterpret_cast<const uint4*>(w_row[t] + (size_t)whole * 2048 + j * 512)
                                     : load16_or_zero(w_row[t] + k + j * 8, in);
#pragma unroll
            for (int m = 0; m < MT; ++m) b[0][m][j].u = load16_or_zero(x_row[m] + k + j * 8, in);
        }
        mma_step(std::integral_constant<int, 0>{});
    }

#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][t * MT + m][lane][i] = acc[t][m][i];
    __shared__ float ssq_red[FUSE == FUSE_RSTD ? WAVES : 1][MT][16];
    if (FUSE == FUSE_RSTD && c == 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m) ssq_red[wave][m][r] = ssq_mine[m];
    }
    __syncthreads();
    float rstd[MT];
    if (FUSE == FUSE_RSTD) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float a = 0.f;
            for (int wv = 0; wv < WAVES; ++wv) a += ssq_red[wv][m][r];
            rstd[m] = 1.0f / sqrtf(a / (float)K + fuse.eps);
        }
    }
    if (GATED) {
        // row tiles come in pairs (gate rows, up rows of the same 16 outputs): the
        // epilogue writes silu(gate) * up, N/2 columns (kernels/src/swiglu_kernel_cpu.cpp:20-24)
        const int n_out = N / 2;
        for (int pair = wave; pair < (RT / 2) * MT; pair += WAVES) {
            const int tp = pair / MT, m = pair % MT;
            float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
            for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    g[i] += red[wv][(2 * tp) * MT + m][lane][i];
                    u[i] += red[wv][(2 * tp + 1) * MT + m][lane][i];
                }
            const int row = m * 16 + r;
            const int n0 = (blockIdx.x * (RT / 2) + tp) * 16 + c * 4;
            if (FUSE == FUSE_RSTD) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    g[i] *= rstd[m];
                    u[i] *= rstd[m];
                }
            }
            if (row < M) {
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = g[i] / (1.0f + expf(-g[i])) * u[i];
                store4(y + (size_t)row * n_out + n0, o, n_out - n0, (n_out & 3) == 0);
            }
        }
        return;
    }
    // tiles are shared out over the waves; each sums the partials in wave order
    for (int tile = wave; tile < RT * MT; tile += WAVES) {
        const int t = tile / MT, m = tile % MT;
        float s[4] = {0.f, 0.f, 0.f, 0.f};
        for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] += red[wv][tile][lane][i];
        const int row = m * 16 + r;
        const int n0 = n_base + t * 16 + c * 4;
        if (FUSE == FUSE_RESIDUAL) {
            // (MT == 1 and tile == wave: the values asked for at the start are this tile's)
            float ssq = 0.f, h[4], hw[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                h[i] = h_old[i] + s[i];
                hw[i] = nw[i] * h[i];
                if (row < M && n0 + i < N) ssq += h[i] * h[i];
            }
            if (row < M) {
                store4(fuse.resid + (size_t)row * N + n0, h, N - n0, (N & 3) == 0);
                store4(fuse.xw + (size_t)row * N + n0, hw, N - n0, (N & 3) == 0);
            }
            ssq = quad_rows_sum(ssq);                  // over the tile's 16 columns
            if (c == 0 && row < M) fuse.ssq_out[(size_t)(blockIdx.x * RT + t) * M + row] = ssq;
            continue;
        }
        if (FUSE == FUSE_RSTD) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] *= rstd[m];
        }
        if (row < M) store4(y + (size_t)row * N + n0, s, N - n0, (N & 3) == 0);
    }
}

#ifndef PIPE_DEPTH
#define PIPE_DEPTH 2
#endif

template <int RT, int MT, int WAVES>
static int launch_skinny(const bf16_t* x, const bf16_t* w, void* y, int M, int N, int K, int y_dtype,
                         int tiled, hipStream_t s) {
    const int blocks = (N + 16 * RT - 1) / (16 * RT);
    constexpr int D = (MT == 1 && RT <= 2) ? PIPE_DEPTH : 2;    // deep prefetch where the registers allow
    if (tiled == 2) {       // gated: pairs of row tiles, silu(gate)*up written as bfloat16
        gemm_skinny_kernel<RT, MT, WAVES, bf16_t, true, true, D><<<blocks, WAVES * 64, 0, s>>>(x, w, (bf16_t*)y, M, N, K, SkinnyFuse{});
    } else if (tiled) {
        if (y_dtype == TLI_BF16)
            gemm_skinny_kernel<RT, MT, WAVES, bf16_t, true, false, D><<<blocks, WAVES * 64, 0, s>>>(x, w, (bf16_t*)y, M, N, K, SkinnyFuse{});
        else
            gemm_skinny_kernel<RT, MT, WAVES, float, true, false, D><<<blocks, WAVES * 64, 0, s>>>(x, w, (float*)y, M, N, K, SkinnyFuse{});
    } else {
        if (y_dtype == TLI_BF16)
            gemm_skinny_kernel<RT, MT, WAVES, bf16_t, false><<<blocks, WAVES * 64, 0, s>>>(x, w, (bf16_t*)y, M, N, K, SkinnyFuse{});
        else
            gemm_skinny_kernel<RT, MT, WAVES, float, false><<<blocks, WAVES * 64, 0, s>>>(x, w, (float*)y, M, N, K, SkinnyFuse{});
    }
    return tli_check_launch("gemm_skinny");
}

template <int MT>
static int pick_skinny(const bf16_t* x, const bf16_t* w, void* y, int M, int N, int K, int y_dtype,
                       int tiled, hipStream_t s, int cfg) {
    // cfg 0: by shape.  Narrow outputs get one 16-column tile per workgroup so that
    // even N = 4096 gives 256 workgroups; wide outputs share x over two tiles.
    const long tiles = (N + 15) / 16;
    if (cfg == 0) cfg = tiles <= tli_compute_units() ? 18 : (tiles < 4 * tli_compute_units() ? 28 : 24);
    if (tiled == 2 && cfg < 20) cfg = 24;          // gated needs pairs of row tiles
    switch (cfg) {
        case 14: return launch_skinny<1, MT, 4>(x, w, y, M, N, K, y_dtype, tiled, s);
        case 18: return launch_skinny<1, MT, 8>(x, w, y, M, N, K, y_dtype, tiled, s);
        case 24: return launch_skinny<2, MT, 4>(x, w, y, M, N, K, y_dtype, tiled, s);
        case 28: return launch_skinny<2, MT, 8>(x, w, y, M, N, K, y_dtype, tiled, s);
        default: return tli_fail("gemm_skinny: unknown configuration %d", cfg);
    }
}

// y[M,N] = x[M,K] . W^T.  `tiled` = 0: w is W[N,K] row-major.  `tiled` = 1: w is the
// same matrix in blocks of 16 rows x 128 columns, zero-padded to whole blocks, stored
// [row block][column block][j = 0..3][lane = 16*c + r][8] with element
// W[16*row block + r][128*column block + 32*c + 8*j + e]: every load instruction of
// a wave then reads 1 KiB in a row.  `tiled` = 2: tiled, and the 16-row blocks alternate
// between a gate matrix and an up matrix (block 2t: gate rows 16t.., block 2t+1: up rows
// 16t..); N counts both, y is [M, N/2] bfloat16 = silu(x.gate^T) * (x.up^T).  cfg 0 picks the launch shape; other values
// (row tiles * 10 + waves) force one, for measurements.
extern "C" int tli_gemm_skinny_bf16(const void* x, const void* w, void* y, int M, int N, int K,
                                    int y_dtype, int tiled, int cfg, void* stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64) return tli_fail("gemm_skinny: %d rows, at most 64", M);
    if (K <= 0 || K % 8) return tli_fail("gemm_skinny: K = %d must be a positive multiple of 8", K);
    if (y_dtype != TLI_BF16 && y_dtype != TLI_F32) return tli_fail("gemm_skinny: bad output dtype %d", y_dtype);
    if (tiled < 0 || tiled > 2) return tli_fail("gemm_skinny: bad layout code %d", tiled);
    if (tiled == 2 && (N % 32 || y_dtype != TLI_BF16))
        return tli_fail("gemm_skinny: a gated product needs N %% 32 == 0 and bfloat16 output");
    if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) return tli_fail("gemm_skinny: operands must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    switch ((M + 15) / 16) {
        case 1: return pick_skinny<1>(xp, wp, y, M, N, K, y_dtype, tiled, s, cfg);
        case 2: return pick_skinny<2>(xp, wp, y, M, N, K, y_dtype, tiled, s, cfg);
        case 3: return pick_skinny<3>(xp, wp, y, M, N, K, y_dtype, tiled, s, cfg);
        default: return pick_skinny<4>(xp, wp, y, M, N, K, y_dtype, tiled, s, cfg);
    }
}

template <int RT, int WAVES>
static int launch_skinny_fused(const bf16_t* x, const bf16_t* w, bf16_t* y, int M, int N, int K, int gated,
                               const SkinnyFuse& f, hipStream_t s) {
    const int blocks = (N + 16 * RT - 1) / (16 * RT);
    if (f.resid)
        gemm_skinny_kernel<RT, 1, WAVES, bf16_t, true, false, PIPE_DEPTH, FUSE_RESIDUAL><<<blocks, WAVES * 64, 0, s>>>(x, w, y, M, N, K, f);
    else if (gated)
        gemm_skinny_kernel<RT, 1, WAVES, bf16_t, true, true, PIPE_DEPTH, FUSE_RSTD><<<blocks, WAVES * 64, 0, s>>>(x, w, y, M, N, K, f);
    else
        gemm_skinny_kernel<RT, 1, WAVES, bf16_t, true, false, PIPE_DEPTH, FUSE_RSTD><<<blocks, WAVES * 64, 0, s>>>(x, w, y, M, N, K, f);
    return tli_check_launch("gemm_skinny (norm taken in)");
}

// The product with a norm taken in (see the top of this file), for up to 16 rows and W in the
// decode layout.  Either  resid != null:  resid[M,N] += x . W^T (float32), xw[M,N] =
// bfloat16(norm_w * resid), ssq_out[ceil(N/16)][M] = partial sums of resid^2 (y is not used);
// or  ssq_in != null:  y = (x . W^T) / sqrt(sum(ssq_in[parts_in][M]) / K + eps), through the
// SwiGLU of a gated matrix if `gated` (y then [M, N/2]).
extern "C" int tli_gemm_skinny_fused_bf16(const void* x, const void* w, void* y, int M, int N, int K, int gated,
                                          const float* ssq_in, int parts_in, float eps, float* resid,
                                          const float* norm_w, void* xw, float* ssq_out, int cfg, void* stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16) return tli_fail("gemm_skinny with a norm: %d rows, at most 16", M);
    if (K <= 0 || K % 8) return tli_fail("gemm_skinny: K = %d must be a positive multiple of 8", K);
    if ((resid != nullptr) == (ssq_in != nullptr))
        return tli_fail("gemm_skinny with a norm: give either the residual to add into or the sums of squares of x");
    if (resid && (gated || !norm_w || !xw || !ssq_out)) return tli_fail("gemm_skinny into the residual: missing arguments");
    if (ssq_in && (parts_in <= 0 || !y)) return tli_fail("gemm_skinny with sums of squares: missing arguments");
    if (gated && N % 32) return tli_fail("gemm_skinny: a gated product needs N %% 32 == 0");
    if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)resid | (uintptr_t)xw) & 15)
        return tli_fail("gemm_skinny: operands must be 16-byte aligned");
    const SkinnyFuse f{ssq_in, parts_in, eps, resid, norm_w, (bf16_t*)xw, ssq_out};
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    const long tiles = (N + 15) / 16;
    if (cfg == 0) cfg = tiles <= tli_compute_units() ? 18 : (tiles < 4 * tli_compute_units() ? 28 : 24);
    if (gated && cfg < 20) cfg = 24;
    switch (cfg) {
        case 14: return launch_skinny_fused<1, 4>(xp, wp, (bf16_t*)y, M, N, K, gated, f, s);
        case 18: return launch_skinny_fused<1, 8>(xp, wp, (bf16_t*)y, M, N, K, gated, f, s);
        case 24: return launch_skinny_fused<2, 4>(xp, wp, (bf16_t*)y, M, N, K, gated, f, s);
        case 28: return launch_skinny_fused<2, 8>(xp, wp, (bf16_t*)y, M, N, K, gated, f, s);
        default: return tli_fail("gemm_skinny: unknown configuration %d", cfg);
    }
}
