// Matrix product for many rows (portions of prompts): y[M,N] = x[M,K] . W^T with W in the
// decode layout (see gemm_skinny.hip), so that a model can do without a row-major copy of
// its weights.  For more than 128 rows the caller (HipOps) takes this kernel or the BLAS
// library's product, whichever it measured faster for the shape: at the layer sizes of
// Qwen3-8B to 32B and 512 to 4,096 rows either is ahead by up to 15% somewhere.
//
// A workgroup owns ROWS rows and 192, 256, 384 or 512 columns and walks all of k in slices of 128:
//   x   each slice [ROWS][128] is copied from memory straight into one of two LDS slots
//       (global_load_lds_dwordx4: lane l of a wave writes the 16 bytes it asked for at LDS
//       base + 16 l), rows swizzled as in gemm_mid.hip (chunk q of row r at q ^ (r & 15));
//       every wave reads all rows from there;
//   W   a wave owns RT column tiles of 16 and takes their fragments from memory into one
//       register stage of four k-steps of 32, each refilled for the next slice as soon as
//       its products have been issued.
// All loads of a wave complete in the order of issue, and every load and every wait for
// one is written in assembly here, so the waits name exact counts: the compiler knows of no
// load of this kernel, and a fragment's wait carries the fragment's registers through so
// that its products come after it.
// (The same kernel on v_mfma_f32_32x32x16_bf16, its W operands put together from pairs of
// these fragments by v_permlane16_swap and v_permlane32_swap, was measured 7% slower.)
//
// Workgroup i runs on die i % 8 (the dies take workgroups in turn): a die is given the row
// blocks of 2,048 rows for one column group, then for the next, so its L2 holds the W panel
// and the rows of x that the workgroups running on it share.
#include "common.h"
#include "gemm_reduce.h"
#include <type_traits>

#pragma clang diagnostic ignored "-Winline-asm"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4r;
typedef __attribute__((address_space(3))) void lds_void_r;

union Pack16r {
    uint4 u;
    u32x4r q;
    bf16x8 v;
};

// f(integral_constant<int, I>) for I = FROM .. TO-1, unrolled at compile time
template <int FROM, int TO, typename F>
__device__ __forceinline__ void rows_static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(std::integral_constant<int, FROM>{});
        rows_static_for<FROM + 1, TO>(f);
    }
}

template <int N>
__device__ __forceinline__ void rows_wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Wait until at most N loads are in flight; the fragments of k-step j depend on it.
template <int N, int RT>
__device__ __forceinline__ void rows_wait_fragments(Pack16r (&a)[RT][4], int j) {
    static_assert(RT == 2 || RT == 3 || RT == 4, "two, three or four column tiles a wave");
    if constexpr (RT == 4)
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a[0][j].q), "+v"(a[1][j].q), "+v"(a[2][j].q), "+v"(a[3][j].q) : "n"(N));
    else if constexpr (RT == 3)
        asm volatile("s_waitcnt vmcnt(%3)" : "+v"(a[0][j].q), "+v"(a[1][j].q), "+v"(a[2][j].q) : "n"(N));
    else
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a[0][j].q), "+v"(a[1][j].q) : "n"(N));
}

// RT column tiles a wave, WAVES waves side by side, MT row tiles (ROWS = 16 MT), x fragments
// taken MH row tiles at a time.  GATED: the column tiles alternate between a gate and an up
// matrix (tiled = 2 of tli_gemm_skinny_bf16) and y is [M, N/2] = silu(gate) * up.
// KG = 2: the workgroup has two such sets of WAVES waves; they take the slices of k in turn (each
// set with LDS slots of its own) and the second set's sums are added to the first's through
// LDS at the end.  Where the outputs alone give one workgroup a compute unit, that puts two
// waves on every SIMD without partial sums in memory.  (The slices of a k range must then be
// even in number.)
template <int RT, int WAVES, int MT, int MH, bool GATED, int KG = 1>
__global__ void __launch_bounds__(WAVES * KG * 64, WAVES * KG == 4 ? 2 : 1)
gemm_rows_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                 float* __restrict__ part, int M, int N, int K, int splits, int slices_per_split) {
    constexpr int ROWS = MT * 16;
    constexpr int SLICE = ROWS * 128;                        // elements of a slice of x
    constexpr int XI = ROWS / (4 * WAVES);                   // copies a wave issues for a slice (64 x 16 bytes each)
    constexpr int HALVES = MT / MH;
    constexpr int BATCHES = 4 * HALVES;                      // batches of x fragments in a slice
    static_assert(ROWS % (4 * WAVES) == 0, "a slice is a whole number of copies for every wave");
    static_assert((4 * WAVES) % 16 == 0, "the swizzle of a lane's chunk is then the same in every copy");
    static_assert(MT % MH == 0 && 3 * RT + XI <= 63, "the wait counts fit the counter");
    extern __shared__ uint4 xs_raw[];
    const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
    // set of waves (the same for a whole wave, and said so: slice numbers follow from it and go into scalar
    // registers), wave in the set
    const int kg = KG == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x / 64) / WAVES);
    const int wave = (int)(threadIdx.x / 64) % WAVES;
    bf16_t* xs = reinterpret_cast<bf16_t*>(xs_raw) + (size_t)kg * 2 * SLICE;     // [2][ROWS][128] for this set, rows swizzled
    const int k_steps = (K + 127) / 128;
    const int n_tiles = (N + 15) / 16;
    // Workgroup i runs on die i % TLI_DIES.  A die takes the row blocks in chunks of 2,048 rows: all
    // row blocks of a chunk for one column group, then for the next column group of the die, and
    // so on; then the next chunk (the x rows of a chunk and a W panel stay in its L2 meanwhile).
    constexpr int CHUNK = 2048 / ROWS;
    const int row_blocks = (M + ROWS - 1) / ROWS;
    const int col_groups = (n_tiles + RT * WAVES - 1) / (RT * WAVES);
    const int groups_a_die = (col_groups + TLI_DIES - 1) / TLI_DIES;
    const int die = blockIdx.x % TLI_DIES, turn = blockIdx.x / TLI_DIES;
    const int chunk = turn / (CHUNK * groups_a_die), in_chunk = turn % (CHUNK * groups_a_die);
    const int chunk_rows = min(CHUNK, row_blocks - chunk * CHUNK);      // row blocks of this chunk (the last may be short)
    // The column groups that do not make a whole round of the eight dies are dealt out by row
    // blocks instead, so that every die gets as many workgroups as the others (5,120 columns are
    // 20 groups of 256: two for every die, and of the other four each die takes half the row
    // blocks of one).
    const int whole = col_groups / TLI_DIES, left = col_groups % TLI_DIES;
    int row_block, col_group;
    if (in_chunk < whole * chunk_rows) {
        row_block = chunk * CHUNK + in_chunk % chunk_rows;
        col_group = (in_chunk / chunk_rows) * TLI_DIES + die;
    } else {
        const int share = (left * chunk_rows + TLI_DIES - 1) / TLI_DIES; // workgroups of the left-over groups a die takes
        const int j = in_chunk - whole * chunk_rows;
        const int at = die * share + j;                                   // index among the left-over groups' workgroups
        if (j >= share || at >= left * chunk_rows) return;                // (the grid is rounded up)
        row_block = chunk * CHUNK + at % chunk_rows;
        col_group = whole * TLI_DIES + at / chunk_rows;
    }
    x += (size_t)row_block * ROWS * K;
    const int n_out = GATED ? N / 2 : N;
    y += (size_t)row_block * ROWS * n_out;
    // with splits > 1 the workgroup walks one of `splits` ranges of k and leaves float32 partial sums
    part += ((size_t)blockIdx.y * M + (size_t)row_block * ROWS) * N;
    M = min(ROWS, M - row_block * ROWS);
    const int slice_begin = blockIdx.y * slices_per_split, slice_end = min(k_steps, slice_begin + slices_per_split);
    const int tile0 = (col_group * WAVES + wave) * RT;

    f32x4 acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // Addresses are a base in scalar registers that moves from slice to slice plus a 32-bit
    // offset that a lane keeps for the whole kernel, so that the loads cost no vector arithmetic.
    // W fragments: block (tile, slice) is 2048 elements, fragment j of this lane at j*512 + lane*8
    // (a tile past the last one reads tile 0 instead: its columns are never stored)
    uint32_t w_off[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
        w_off[t] = (uint32_t)(((size_t)(tile0 + t < n_tiles ? tile0 + t : 0) * k_steps * 2048 + lane * 8) * sizeof(bf16_t));
    Pack16r a[RT][4];
    auto load_w = [&](int slice, int j) {          // (j is a constant wherever this is called: one branch remains)
        const uint64_t base = (uint64_t)(uintptr_t)w + (uint64_t)slice * 4096u;
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            if (j == 0) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(a[t][0].q) : "v"(w_off[t]), "s"(base));
            if (j == 1) asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(a[t][1].q) : "v"(w_off[t]), "s"(base));
            if (j == 2) asm volatile("global_load_dwordx4 %0, %1, %2 offset:2048" : "=v"(a[t][2].q) : "v"(w_off[t]), "s"(base));
            if (j == 3) asm volatile("global_load_dwordx4 %0, %1, %2 offset:3072" : "=v"(a[t][3].q) : "v"(w_off[t]), "s"(base));
        }
    };
    // What this lane asks for in copy e of a slice: LDS place (e WAVES + wave) 64 + lane, that is
    // row place / 16 and the chunk that belongs at chunk place % 16 of that row.  Rows past M
    // repeat the last row (never stored).  Where K is no multiple of 128 the columns past K of
    // the last slice read the row's first 8 columns instead (they meet the zeros that pad W).
    const int x_row0 = wave * 4 + lane / 16;
    const int x_col = ((lane % 16) ^ (x_row0 & 15)) * 8;
    uint32_t x_off[XI];
#pragma unroll
    for (int e = 0; e < XI; ++e)
        x_off[e] = (uint32_t)(((size_t)min(x_row0 + e * 4 * WAVES, M - 1) * K + x_col) * sizeof(bf16_t));
    const uint32_t xs_base = (uint32_t)(uintptr_t)(lds_void_r*)xs + (uint32_t)wave * 1024u;
    const bool ragged = (K & 127) != 0;
    // the slot of a slice: the sets of waves take slices in turn, a set's slices alternate between its two slots
    auto slot_of = [&](int slice) { return ((slice - slice_begin) / KG) & 1; };
    auto copy_x = [&](int slice) {
        const uint32_t slot_base = xs_base + (uint32_t)slot_of(slice) * (SLICE * 2);
        if (ragged && slice == k_steps - 1) {          // (the last slice of the last range)
            const int k = slice * 128 + x_col;
#pragma unroll
            for (int e = 0; e < XI; ++e) {
                const bf16_t* src = x + (size_t)min(x_row0 + e * 4 * WAVES, M - 1) * K + (k < K ? k : 0);
                const uint32_t dst = __builtin_amdgcn_readfirstlane(slot_base + (uint32_t)(e * WAVES * 1024));
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src) : "m0", "memory");
            }
            return;
        }
        const uint64_t base = (uint64_t)(uintptr_t)x + (uint64_t)slice * 256u;
#pragma unroll
        for (int e = 0; e < XI; ++e) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(slot_base + (uint32_t)(e * WAVES * 1024));
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(x_off[e]), "s"(base) : "m0", "memory");
        }
    };
    // LDS offsets of this lane's x fragments: row m*16 + r, chunk (4c + j) ^ r
    int b_col[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b_col[j] = r * 128 + ((4 * c + j) ^ r) * 8;

    // batch n of a slice: k-step j = n / HALVES, row tiles (n % HALVES) * MH ..; batch n + 1 is
    // read from LDS before batch n is multiplied
    Pack16r b[2][MH];
    auto read_b = [&](int slice, int n, Pack16r (&dst)[MH]) {
        const bf16_t* xb = xs + slot_of(slice) * SLICE;
        const int j = n / HALVES, h = n % HALVES;
#pragma unroll
        for (int m = 0; m < MH; ++m)
            dst[m].u = *reinterpret_cast<const uint4*>(xb + (h * MH + m) * 16 * 128 + b_col[j]);
    };
    auto multiply = [&](int n, Pack16r (&src)[MH]) {
        const int j = n / HALVES, h = n % HALVES;
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int m = 0; m < MH; ++m)
                acc[t][h * MH + m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][j].v, src[m].v, acc[t][h * MH + m], 0, 0, 0);
    };
    // Loads in flight behind the fragments of k-step j when they are waited for: the k-steps
    // after j of this slice (3 - j times RT), the copy of the next slice of x (XI) and the
    // k-steps before j of the next slice (j times RT): 3 RT + XI for every j.  In the last slice
    // nothing follows: (3 - j) RT.
    auto one_slice = [&](int slice, auto LAST_T) {
        constexpr bool LAST = decltype(LAST_T)::value;
        read_b(slice, 0, b[0]);
        rows_static_for<0, BATCHES>([&](auto N_T) {
            constexpr int n = decltype(N_T)::value, j = n / HALVES;
            if constexpr (n % HALVES == 0) {
                if constexpr (LAST)
                    rows_wait_fragments<(3 - j) * RT, RT>(a, j);
                else
                    rows_wait_fragments<3 * RT + XI, RT>(a, j);
            }
            if constexpr (n + 1 < BATCHES) read_b(slice, n + 1, b[(n + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            multiply(n, b[n & 1]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!LAST && n % HALVES == HALVES - 1) load_w(slice + KG, j);
        });
    };

    if (slice_begin < slice_end) {
        int slice = slice_begin + kg;
        copy_x(slice);
        load_w(slice, 0);
        load_w(slice, 1);
        load_w(slice, 2);
        load_w(slice, 3);
        for (; slice + KG < slice_end; slice += KG) {
            rows_wait_loads<4 * RT>();     // this wave's part of the slice of x has landed (behind it: 4 RT fragments)
            __syncthreads();               // everyone's has, and everyone has finished the slice before
            copy_x(slice + KG);            // into the slot that the slice before used
            one_slice(slice, std::false_type{});
        }
        rows_wait_loads<4 * RT>();
        __syncthreads();
        one_slice(slice, std::true_type{});
    }
    if constexpr (KG == 2) {
        // the second set hands its sums over: [wave][accumulator][lane] of 16 bytes, as much as
        // the four slots of x together
        static_assert(KG == 1 || RT * MT * 64 * 16 * WAVES <= 2 * 2 * SLICE * 2, "the sums fit the slots of x");
        __syncthreads();                   // nobody reads x any more
        f32x4* sums = reinterpret_cast<f32x4*>(xs_raw) + (size_t)wave * RT * MT * 64 + lane;
        if (kg == 1) {
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m) sums[(t * MT + m) * 64] = acc[t][m];
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const f32x4 other = sums[(t * MT + m) * 64];
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][m][i] += other[i];
            }
    }

    if (splits > 1) {
        // partial sums [split][row][column of W as tiled]: the pass that adds them knows a gated layout
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            const int n0 = (tile0 + t) * 16 + 4 * c;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = m * 16 + r;
                if (row >= M) continue;
                float* dst = part + (size_t)row * N + n0;
                if (n0 + 3 < N && N % 4 == 0) {
                    *reinterpret_cast<f32x4*>(dst) = acc[t][m];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < N) dst[i] = acc[t][m][i];
                }
            }
        }
        return;
    }
    // lane holds y[m*16 + r][tile*16 + 4c + i]
    if (GATED) {
        // one output tile from a gate tile's sums and its up tile's: silu(g) * u with the hardware's exp2 and
        // reciprocal (1 ulp each; the result is rounded to bfloat16): the library routines would cost more
        // vector instructions here than the workgroup's MFMAs
        auto store_pair = [&](const f32x4 (&gate)[MT], const f32x4 (&up)[MT], int gate_tile) {
            const int n0 = (gate_tile / 2) * 16 + 4 * c;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = m * 16 + r;
                if (row >= M) continue;
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g = gate[m][i], u = up[m][i];
                    o[i] = g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g)) * u;
                }
                bf16_t* dst = y + (size_t)row * n_out + n0;
                if (n0 + 3 < n_out && n_out % 4 == 0) {
                    *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < n_out) dst[i] = f32_to_bf16(o[i]);
                }
            }
        };
        if constexpr (RT % 2 == 0) {
#pragma unroll
            for (int t = 0; t + 1 < RT; t += 2) store_pair(acc[t], acc[t + 1], tile0 + t);
        } else {
            // Three tiles a wave: a workgroup's tiles start at an even one (gate), so an even wave holds
            // gate, up, gate and the odd wave after it up, gate, up.  The odd wave hands the sums of its
            // first tile over through LDS, [pair of waves][row tile][lane] of 16 bytes, to the even wave,
            // which holds their gate tile.
            static_assert(RT == 3 && WAVES % 2 == 0 && KG == 1, "pairs of waves share a gate and an up tile");
            static_assert((WAVES / 2) * MT * 64 * 16 <= 2 * SLICE * 2, "the sums fit the slots of x");
            __syncthreads();                   // nobody reads x any more
            f32x4* sums = reinterpret_cast<f32x4*>(xs_raw) + (size_t)(wave / 2) * MT * 64 + lane;
            if (wave % 2 == 1) {
#pragma unroll
                for (int m = 0; m < MT; ++m) sums[m * 64] = acc[0][m];
            }
            __syncthreads();
            if (wave % 2 == 0) {
                f32x4 up[MT];
#pragma unroll
                for (int m = 0; m < MT; ++m) up[m] = sums[m * 64];
                store_pair(acc[0], acc[1], tile0);
                store_pair(acc[2], up, tile0 + 2);
            } else {
                store_pair(acc[1], acc[2], tile0 + 1);
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int n0 = (tile0 + t) * 16 + 4 * c;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = m * 16 + r;
            if (row >= M) continue;
            bf16_t* dst = y + (size_t)row * N + n0;
            if (n0 + 3 < N && N % 4 == 0) {
                *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(acc[t][m][0], acc[t][m][1]),
                                                            pack_bf16x2(acc[t][m][2], acc[t][m][3]));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n0 + i < N) dst[i] = f32_to_bf16(acc[t][m][i]);
            }
        }
    }
}

template <int RT, int WAVES, int MT, int MH, int KG = 1>
static int launch_rows(const bf16_t* x, const bf16_t* w, bf16_t* y, float* part, int M, int N, int K, int gated,
                       int splits, hipStream_t s) {
    const int n_tiles = (N + 15) / 16, k_steps = (K + 127) / 128;
    const long col_groups = (n_tiles + RT * WAVES - 1) / (RT * WAVES), row_blocks = (M + MT * 16 - 1) / (MT * 16);
    const long chunk = 2048 / (MT * 16);                     // as the kernel deals the row blocks out
    const long blocks = (col_groups + TLI_DIES - 1) / TLI_DIES * TLI_DIES * ((row_blocks + chunk - 1) / chunk * chunk);
    if (blocks > 2147483647L) return tli_fail("gemm_rows: too many workgroups");
    const int slices_per_split = (k_steps + splits - 1) / splits;
    if (KG == 2 && (slices_per_split % 2 || k_steps % slices_per_split))
        return tli_fail("gemm_rows: two sets of waves need an even number of slices in every range of k (%d of %d)",
                        slices_per_split, k_steps);
    const dim3 grid((unsigned)blocks, (unsigned)splits);
    const size_t lds = (size_t)KG * 2 * MT * 16 * 128 * sizeof(bf16_t);
    // (more than 64 KiB of LDS has to be allowed for a kernel once)
#define ROWS_LAUNCH(G)                                                                                     \
    {                                                                                                      \
        auto kernel = gemm_rows_kernel<RT, WAVES, MT, MH, G, KG>;                                          \
        static bool allowed = false;                                                                       \
        if (lds > 65536 && !allowed) {                                                                     \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,       \
                                    (int)lds) != hipSuccess)                                               \
                return tli_fail("gemm_rows: cannot have %zu bytes of LDS", lds);                           \
            allowed = true;                                                                                \
        }                                                                                                  \
        kernel<<<grid, WAVES * KG * 64, lds, s>>>(x, w, y, part, M, N, K, splits, slices_per_split);       \
    }
    if (gated) ROWS_LAUNCH(true)
    else ROWS_LAUNCH(false)
#undef ROWS_LAUNCH
    if (tli_check_launch("gemm_rows")) return 1;
    if (splits > 1 && y) {
        launch_gemm_reduce(part, y, M, N, splits, gated, s);
        return tli_check_launch("gemm_rows: sum of the partial products");
    }
    return 0;
}

// How many ranges of k a product of this shape is cut into (the caller sizes `part` by it):
// until there are about three workgroups for every four compute units, a range keeping at
// least four slices of 128.
extern "C" int tli_gemm_rows_splits(int M, int N, int K) {
    const long col_groups = ((N + 15) / 16 + 15) / 16, row_blocks = (M + 127) / 128;
    const int k_steps = (K + 127) / 128;
    int splits = 1;
    const long enough = 3L * tli_compute_units() / 4;
    while (col_groups * row_blocks * splits < enough && splits * 2 * 4 <= k_steps && splits < 16) splits *= 2;
    return splits;
}

// The launch shape that cfg 0 takes: the one whose workgroups fill the 256 compute units best.
// What a shape costs is counted in rounds of workgroups on a die (the kernel deals the
// workgroups out evenly over the eight dies of 32 compute units), from measurements at the
// layer sizes of Qwen3-8B to 32B and 256 to 8,192 rows.  With four waves a workgroup two
// workgroups share a compute unit and each then takes 1.75 times as long as alone, so up to 32
// workgroups a die cost one unit, up to 64 cost 1.75, and every further 64 as much again (a
// remainder of up to 32 one unit); 128 x 192 outputs cost 6% more a column than 128 x 256 but divide 6,144 or 5,120
// columns over the chip where 256 leave a quarter of it idle.  128 x 512 outputs in eight
// waves, one workgroup a compute unit, ask the L2 caches for a sixth less: 0.84 a column, in
// rounds of 32 workgroups a die.  128 x 256 outputs by two sets of four waves that share out the
// slices of k (one workgroup a compute unit again) cost 0.88 of what four waves alone do, and a
// good deal less where k is cut into ranges as well; only for an even number of slices.
static int rows_pick(int M, int N, int K, int splits, int gated) {
    const long n_tiles = (N + 15) / 16, row_blocks = (M + 127) / 128;
    // workgroups of the busiest of the eight dies (each has 32 compute units), in units of one
    // workgroup alone on its compute unit
    const long units = tli_units_a_die();          // compute units of a die (32)
    auto a_die = [&](long tiles_a_group) { return ((n_tiles + tiles_a_group - 1) / tiles_a_group * row_blocks * splits + TLI_DIES - 1) / TLI_DIES; };
    auto shared = [&](long wgs) {                  // four waves a workgroup: two workgroups share a compute unit
        if (wgs <= units) return 1.0;
        const long full = wgs / (2 * units), rem = wgs % (2 * units);
        return 1.75 * (double)full + (rem == 0 ? 0.0 : rem <= units ? 1.0 : 1.75);
    };
    auto alone = [&](long wgs) { return (double)((wgs + units - 1) / units); };     // eight waves: one workgroup a compute unit
    const long k_steps = (K + 127) / 128, per = (k_steps + splits - 1) / splits;
    const double cost2 = shared(a_die(16)) * 256.0, cost4 = shared(a_die(12)) * 192.0 * 1.06;
    const double cost3 = alone(a_die(32)) * 512.0 * 0.84, cost6 = alone(a_die(16)) * 256.0 * 0.88;
    // 128 x 384 outputs in eight waves of three column tiles (one workgroup a compute unit): 0.82 a
    // column; 5,120 columns are 14 such groups, 6,144 are 16, the 24,576 of a gate/up pair of 12,288 are 64
    const double cost5 = alone(a_die(24)) * 384.0 * 0.82;
    // (from three rounds of the 512-column shape on, it was the fastest at every layer size measured:
    // the costs above are those of the first rounds.  A gated product counts whole rounds only: with
    // two and a bit, the shapes that divide its many columns evenly were 12 to 14% faster)
    if (gated ? a_die(32) >= 3 * units : alone(a_die(32)) >= 3.0) return 3;
    int best = 2;
    double cost = cost2;
    if (cost3 < cost) { best = 3; cost = cost3; }
    if (cost4 < cost) { best = 4; cost = cost4; }
    if (cost5 < cost) { best = 5; cost = cost5; }
    if (!gated && per % 2 == 0 && k_steps % per == 0 && cost6 < cost) best = 6;
    return best;
}

// y[M,N] = x[M,K] . W^T for any number of rows, bfloat16, W in the decode layout (`gated` as
// tiled = 2 of tli_gemm_skinny_bf16: N counts gate and up, y is [M, N/2]).  `part`: splits*M*N
// floats when splits > 1 (splits as returned by tli_gemm_rows_splits, or forced by the
// caller); with y null the partial sums [splits][M][N] are left for the consumer to add
// (tli_gemm_mid_reduce, or tli_add_rmsnorm).
// cfg 0 picks the launch shape; 1: 256 x 256 outputs a workgroup of eight waves, 2: 128 x 256
// and four waves, two workgroups a compute unit, 3: 128 x 512 and eight waves, 4: 128 x 192 and
// four waves, 5: 128 x 384 and eight waves (in a gated product the waves of 4 and 5, which hold three
// column tiles each, exchange the sums of one tile in pairs), 6: 128 x 256
// by two sets of four waves that take the slices of k in turn; cfg >= 10: the tens for a gated product, the
// ones for the others (measurements).
extern "C" int tli_gemm_rows_bf16(const void* x, const void* w, void* y, float* part, int M, int N, int K,
                                  int gated, int splits, int cfg, void* stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || K % 8) return tli_fail("gemm_rows: K = %d must be a positive multiple of 8", K);
    if (gated && N % 32) return tli_fail("gemm_rows: a gated product needs N %% 32 == 0");
    if (!x || !w) return tli_fail("gemm_rows: null operand");
    if (splits < 1 || splits > 64) return tli_fail("gemm_rows: %d splits", splits);
    if (splits > 1 && !part) return tli_fail("gemm_rows: splits need a buffer for partial sums");
    if (!y && (splits < 2 || gated)) return tli_fail("gemm_rows: only a plain product with split k can leave its partial sums");
    if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)part) & 15) return tli_fail("gemm_rows: operands must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    if ((size_t)M * K * sizeof(bf16_t) >= (1ull << 32) || (size_t)((N + 15) / 16 * 16) * ((K + 127) / 128 * 128) * sizeof(bf16_t) >= (1ull << 32))
        return tli_fail("gemm_rows: an operand of 4 GiB or more (offsets are 32 bits)");
    if (cfg >= 10) cfg = gated ? cfg / 10 : cfg % 10;       // measurements: one shape for the gated product, one for the others
    if (cfg == 0) cfg = rows_pick(M, N, K, splits, gated);
    if (cfg == 1) return launch_rows<2, 8, 16, 1>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    if (cfg == 2) return launch_rows<4, 4, 8, 1>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    if (cfg == 3) return launch_rows<4, 8, 8, 1>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    if (cfg == 6) {
        const int k_steps = (K + 127) / 128, per = (k_steps + splits - 1) / splits;
        if (per % 2 || k_steps % per) cfg = 2;       // (an odd number of slices somewhere: one set of waves)
        else return launch_rows<4, 4, 8, 1, 2>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    }
    if (cfg == 2) return launch_rows<4, 4, 8, 1>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    if (cfg == 4) {
        return launch_rows<3, 4, 8, 1>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    }
    if (cfg == 5) {
        return launch_rows<3, 8, 8, 1>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, part, M, N, K, gated, splits, s);
    }
    return tli_fail("gemm_rows: unknown configuration %d", cfg);
}
