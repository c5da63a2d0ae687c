// Matrix product for 17..128 rows (a large decode batch), and for plain products of up to 256: y[M,N] =
// x[M,K] . W^T with W in the decode layout (see gemm_skinny.hip).  Still bound by streaming W once, but with
// four or eight 16-row tiles of x every W fragment meets as many x fragments, and taking
// those from L2 for every wave (as the kernel for <= 16 rows does) would cost that many
// times the traffic of W itself.  Here the waves of a workgroup own different output
// columns and walk k together: each 128-wide slice of x (16 MT rows, 4 MT KiB) is brought
// into LDS once and shared by all of them.
//
// The slices of x are copied from memory straight into a ring of LDS buffers
// (global_load_lds_dwordx4: lane l of a wave writes the 16 bytes it asked for at LDS
// base + 16 l), DEPTH + 1 slices ahead; the W fragments go into a ring of register
// stages, DEPTH slices ahead.  No register holds x on its way, and one barrier a slice
// is enough.  Such a copy leaves no room for padding between rows, so the rows are
// swizzled: the 16-byte chunk q of row r lies at chunk q ^ (r & 15), and a lane asks for
// the chunk that belongs at its place; the 16 lanes that read one chunk column of 16
// rows for an MFMA operand then hit 16 different bank groups.
//
// A workgroup owns 16*RT*WAVES output columns and one of `splits` contiguous ranges
// of k.  With splits > 1 it writes float32 partial sums [split][M][N] and a second
// small kernel adds them in split order (and applies the SwiGLU epilogue for a gated
// matrix), so the result does not depend on timing.  (Letting the workgroup that
// finishes last do the sum inside the same kernel was measured and is much slower: the
// eight L2 caches of the chip are not coherent with each other, so publishing partial
// sums between workgroups costs a write-back and an invalidation in every workgroup;
// the kernel boundary does both once.)
#include "common.h"
#include "gemm_reduce.h"
#include <type_traits>

// (the copies below set m0 in assembly and say so; nothing else in this file uses m0)
#pragma clang diagnostic ignored "-Winline-asm"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4m;
typedef __attribute__((address_space(3))) void lds_void_m;

union Pack16m {
    uint4 u;
    u32x4m q;
    bf16x8 v;
};

#define MID_MAX_ROWS 256

template <int RT, int WAVES, int DEPTH, int MT, typename TO, bool GATED>
__global__ void __launch_bounds__(WAVES * 64)
gemm_mid_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, TO* __restrict__ y,
                float* __restrict__ part, int M_all, int N, int K, int splits, int steps_per_split) {
    constexpr int ROWS = MT * 16;
    constexpr int STAGES = DEPTH + 1;                        // W: DEPTH slices on their way, one in use
    constexpr int XSLOTS = DEPTH + 2;                        // x: one slice further ahead
    constexpr int SLICE = ROWS * 128;                        // elements of a slice of x
    constexpr int COPIES = ROWS / 4;                         // copies of 64 x 16 bytes that make up a slice
    // copies a wave issues for a slice: the same number for every wave (where the waves do not divide
    // the copies, the last one is made again by the waves that would have none)
    constexpr int XI = (COPIES + WAVES - 1) / WAVES;
    extern __shared__ uint4 xs_raw[];
    bf16_t* xs = reinterpret_cast<bf16_t*>(xs_raw);          // [XSLOTS][ROWS][128], rows swizzled
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, r = lane % 16, c = lane / 16;
    const int k_steps = (K + 127) / 128;
    const int n_tiles = (N + 15) / 16;
    // More than ROWS rows: the row blocks of one column group are workgroups 8 apart, which run on the
    // same die at the same time, so that the second one finds the W fragments in that die's L2.
    const int row_blocks = (M_all + ROWS - 1) / ROWS;
    int group = blockIdx.x, row0 = 0;
    if (row_blocks > 1) {
        row0 = (group / TLI_DIES) % row_blocks * ROWS;
        group = group / (TLI_DIES * row_blocks) * TLI_DIES + group % TLI_DIES;
        if (group * WAVES * RT >= n_tiles) return;            // (the column groups are rounded up to a multiple of 8)
    }
    const int M = min(ROWS, M_all - row0);
    x += (size_t)row0 * K;
    const int tile0 = (group * WAVES + wave) * RT;            // this wave's first 16-column tile
    const int step_begin = blockIdx.y * steps_per_split;
    const int step_end = min(k_steps, step_begin + steps_per_split);
    // Workgroups walk their k range from different starting slices, wrapping round: a
    // slice of x is rows a power of two apart, which all lie in one channel of the L2
    // cache, and workgroups in step would all wait for that one channel.  (Workgroups go
    // round the eight dies in turn, so neighbours on a die are blockIdx.x / 8 apart.)
    const int rot = step_begin < step_end ? (group / TLI_DIES) % (step_end - step_begin) : 0;
    auto at = [&](int step) { return step + rot < step_end ? step + rot : step + rot - (step_end - step_begin); };

    f32x4 acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // W fragments straight from the decode layout: block (tile, step) is 2048 elements,
    // fragment j of this lane at j*512 + lane*8
    // (a tile past the last one reads tile 0 instead: its columns are never stored.  No
    // load below is predicated: a branch around a load makes the compiler wait for every
    // load in flight at the next use, which would undo the prefetching)
    const bf16_t* w_tile[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
        w_tile[t] = w + (size_t)(tile0 + t < n_tiles ? tile0 + t : 0) * k_steps * 2048 + lane * 8;
    Pack16m a[STAGES][RT][4];
    auto fetch_w = [&](int logical, auto STAGE) {
        constexpr int S = decltype(STAGE)::value;
        const int step = at(logical);
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                // (read once a step, a whole KiB an instruction: not to be kept by the caches, which
                // hold what every kernel begins with; see gemm_skinny.hip)
                a[S][t][j].q = __builtin_nontemporal_load(reinterpret_cast<const u32x4m*>(w_tile[t] + (size_t)step * 2048 + j * 512));
    };
    // What this lane asks for in copy e of a slice: LDS place (e WAVES + wave) 64 + lane, that
    // is row place / 16 and the chunk that belongs at chunk place % 16 of that row.  Rows past
    // M repeat the last row (never stored); columns past K read the row's first 8 columns
    // instead (they meet the zeros that pad W).
    const bf16_t* x_row[XI];
    int x_col[XI];
    uint32_t x_dst[XI];                                      // where copy e lands in a slot (bytes)
#pragma unroll
    for (int e = 0; e < XI; ++e) {
        const int copy = min(e * WAVES + wave, COPIES - 1);
        const int place = copy * 64 + lane, row = place / 16;
        x_row[e] = x + (size_t)min(row, M - 1) * K;
        x_col[e] = ((place % 16) ^ (row & 15)) * 8;
        x_dst[e] = (uint32_t)copy * 1024u;
    }
    // (The copy is written in assembly: told of it, the compiler waits for every load in
    // flight before the next LDS read, because the copy writes LDS.  Untold, it counts
    // fewer loads in flight than there are when it waits for W fragments, and so waits for
    // somewhat more than it needs: for the copies issued before the fragments it lets fly.)
    const uint32_t xs_base = (uint32_t)(uintptr_t)(lds_void_m*)xs;
    auto fetch_x = [&](int logical) {
        const int step = at(logical);
        const uint32_t slot_base = xs_base + (uint32_t)((logical - step_begin) % XSLOTS) * (SLICE * 2);
#pragma unroll
        for (int e = 0; e < XI; ++e) {
            const int k = step * 128 + x_col[e];
            const bf16_t* src = x_row[e] + (k < K ? k : 0);
            const uint32_t dst = __builtin_amdgcn_readfirstlane(slot_base + x_dst[e]);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         :: "s"(dst), "v"(src) : "m0");
        }
    };
    // Loads complete in the order of issue, and the copy of slice s+1 of x is issued before
    // the W fragments of slice s: a wave that has multiplied slice s (it waited for those
    // fragments) has its part of slice s+1 of x in LDS, and after the barrier that opens
    // slice s+1 every wave has.  (The scheduling barriers keep the compiler from changing
    // the order of issue.)
    auto fetch = [&](int logical, auto STAGE, bool with_x) {
        if (with_x) fetch_x(logical + 1);
        __builtin_amdgcn_sched_barrier(0);
        fetch_w(logical, STAGE);
        __builtin_amdgcn_sched_barrier(0);
    };
    // LDS offsets of this lane's x fragments: row m*16 + r, chunk (4c + j) ^ r
    int b_col[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b_col[j] = r * 128 + ((4 * c + j) ^ r) * 8;

    // one slice: `step` is multiplied from W stage S and the LDS slot of its x.  FULL: the
    // fetches of this round exist, so they are under no branch (after a branch that may have
    // issued loads the compiler waits as if it had not, that is for all of them)
    auto slice = [&](int step, auto STAGE, auto FULL_T) {
        constexpr int S = decltype(STAGE)::value;
        constexpr bool FULL = decltype(FULL_T)::value;
        __syncthreads();        // everyone's part of this slice of x is in LDS, and everyone has finished the slice before
        if (FULL || step + DEPTH < step_end)
            fetch(step + DEPTH, std::integral_constant<int, (S + DEPTH) % STAGES>{}, FULL || step + DEPTH + 1 < step_end);
        const bf16_t* xb = xs + ((step - step_begin) % XSLOTS) * SLICE;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            Pack16m b[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m)
                b[m].u = *reinterpret_cast<const uint4*>(xb + m * 16 * 128 + b_col[j]);
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[S][t][j].v, b[m].v, acc[t][m], 0, 0, 0);
        }
    };
    auto slices = [&](auto self, int step, auto INDEX, auto FULL_T) -> void {
        constexpr int I = decltype(INDEX)::value;
        if constexpr (I < STAGES) {
            if (decltype(FULL_T)::value || step + I < step_end) {
                slice(step + I, std::integral_constant<int, I>{}, FULL_T);
                self(self, step, std::integral_constant<int, I + 1>{}, FULL_T);
            }
        }
    };
    auto prologue = [&](auto self, auto INDEX) -> void {
        constexpr int I = decltype(INDEX)::value;
        if constexpr (I < DEPTH) {
            if (step_begin + I < step_end)
                fetch(step_begin + I, std::integral_constant<int, I>{}, step_begin + I + 1 < step_end);
            self(self, std::integral_constant<int, I + 1>{});
        }
    };

    if (step_begin < step_end) {
        fetch_x(step_begin);
        prologue(prologue, std::integral_constant<int, 0>{});
        // the first slice of x has no W fragments behind it that anyone waits for before the
        // first barrier: wait for it here
        __builtin_amdgcn_s_waitcnt(0x0F70);             // vmcnt(0)
    }
    int step = step_begin;
    for (; step + STAGES - 1 + DEPTH + 1 < step_end; step += STAGES)
        slices(slices, step, std::integral_constant<int, 0>{}, std::true_type{});
    for (; step < step_end; step += STAGES)
        slices(slices, step, std::integral_constant<int, 0>{}, std::false_type{});

    // lane holds y[m*16 + r][tile*16 + 4c + i]
    if (splits > 1) {
        float* dst = part + ((size_t)blockIdx.y * M_all + row0) * N;
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            const int n0 = (tile0 + t) * 16 + 4 * c;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = m * 16 + r;
                if (row >= M) continue;
                if (n0 + 3 < N && (N & 3) == 0) {           // (the lane's four sums in one store)
                    *reinterpret_cast<f32x4*>(dst + (size_t)row * N + n0) = acc[t][m];
                    continue;
                }
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n0 + i < N) dst[(size_t)row * N + n0 + i] = acc[t][m][i];
            }
        }
        return;
    }
    if (GATED) {
        const int n_out = N / 2;
        y += (size_t)row0 * n_out;
#pragma unroll
        for (int t = 0; t + 1 < RT; t += 2) {
            const int n0 = ((tile0 + t) / 2) * 16 + 4 * c;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = m * 16 + r;
                if (row >= M) continue;
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g = acc[t][m][i], u = acc[t + 1][m][i];
                    o[i] = g / (1.0f + expf(-g)) * u;
                }
                store4(y + (size_t)row * n_out + n0, o, n_out - n0, (n_out & 3) == 0);
            }
        }
        return;
    }
    y += (size_t)row0 * N;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int n0 = (tile0 + t) * 16 + 4 * c;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = m * 16 + r;
            if (row >= M) continue;
            const float o[4] = {acc[t][m][0], acc[t][m][1], acc[t][m][2], acc[t][m][3]};
            store4(y + (size_t)row * N + n0, o, N - n0, (N & 3) == 0);
        }
    }
}

template <int RT, int WAVES, int DEPTH, int MT>
static int launch_mid_rows(const bf16_t* x, const bf16_t* w, void* y, float* part, int M, int N, int K,
                           int y_dtype, int gated, int splits, hipStream_t s) {
    const int n_tiles = (N + 15) / 16, k_steps = (K + 127) / 128;
    const int steps_per_split = (k_steps + splits - 1) / splits;
    const int groups = (n_tiles + RT * WAVES - 1) / (RT * WAVES), row_blocks = (M + MT * 16 - 1) / (MT * 16);
    dim3 grid(row_blocks > 1 ? (groups + TLI_DIES - 1) / TLI_DIES * TLI_DIES * row_blocks : groups, splits);
    const size_t lds = (size_t)(DEPTH + 2) * MT * 16 * 128 * sizeof(bf16_t);
    // (more than 64 KiB of LDS has to be allowed for a kernel once)
#define MID_LAUNCH(TO, G)                                                                                  \
    {                                                                                                      \
        auto kernel = gemm_mid_kernel<RT, WAVES, DEPTH, MT, TO, G>;                                        \
        static bool allowed = false;                                                                       \
        if (lds > 65536 && !allowed) {                                                                     \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,       \
                                    (int)lds) != hipSuccess)                                               \
                return tli_fail("gemm_mid: cannot have %zu bytes of LDS", lds);                            \
            allowed = true;                                                                                \
        }                                                                                                  \
        kernel<<<grid, WAVES * 64, lds, s>>>(x, w, (TO*)y, part, M, N, K, splits, steps_per_split);        \
    }
    if (gated) MID_LAUNCH(bf16_t, true)
    else if (y_dtype == TLI_BF16) MID_LAUNCH(bf16_t, false)
    else MID_LAUNCH(float, false)
#undef MID_LAUNCH
    if (tli_check_launch("gemm_mid")) return 1;
    if (splits > 1 && y) {
        if (y_dtype == TLI_BF16) launch_gemm_reduce(part, (bf16_t*)y, M, N, splits, gated, s);
        else launch_gemm_reduce(part, (float*)y, M, N, splits, gated, s);
        return tli_check_launch("gemm_mid_reduce");
    }
    return 0;
}

// Four 16-row tiles of x up to 64 rows, eight beyond.
template <int RT, int WAVES, int DEPTH>
static int launch_mid(const bf16_t* x, const bf16_t* w, void* y, float* part, int M, int N, int K,
                      int y_dtype, int gated, int splits, hipStream_t s) {
    if (M <= 64) return launch_mid_rows<RT, WAVES, DEPTH, 4>(x, w, y, part, M, N, K, y_dtype, gated, splits, s);
    if constexpr (DEPTH <= 3)       // (DEPTH + 2) slices of 32 KiB fit the 160 KiB of LDS
        return launch_mid_rows<RT, WAVES, DEPTH, 8>(x, w, y, part, M, N, K, y_dtype, gated, splits, s);
    else
        return tli_fail("gemm_mid: more than 64 rows leave LDS for at most 3 slices on their way");
}

// Launch shape by measurement on MI355X (4096..151936 columns, k of 4096..25600): two
// column tiles a wave once that still leaves about 192 workgroups, else one; k is cut into
// ranges until there are about 192 workgroups (tli_gemm_mid_bf16 then keeps the workgroups
// at no more than one a compute unit where it can).
static int mid_tiles_per_wave(int N, int gated) { return gated || (N + 15) / 16 >= 8 * (3 * tli_compute_units() / 4) ? 2 : 1; }

// How a product of this shape is dealt out: column tiles a wave and ranges of k.  As many
// workgroups as fit the 256 compute units once (more cost more than they bring, measured at
// the layer sizes of Qwen3-8B to 32B): with one tile a wave (four waves: 64 columns a workgroup)
// as many ranges as that allows, 5,120 columns in 3 ranges (240 workgroups; 4 ranges of 128
// columns, 160 workgroups, were 9% slower); where the columns alone are more than 128 groups
// but fewer than 192, two tiles a wave and the ranges that go with them (10,240 columns: 80
// groups in 3 ranges).  A range keeps at least two slices of 128.  Gated products: see below.
static void mid_plan(int N, int K, int gated, int row_blocks, int* tiles_a_wave, int* waves_a_group, int* ranges) {
    const int n_tiles = (N + 15) / 16, k_steps = (K + 127) / 128;
    const int units = tli_compute_units(), most = 3 * units / 4;      // 256 and 192 on MI355X
    if (row_blocks > 1) {
        // Row blocks of 128 rows side by side (the second finds the W fragments in its die's L2): two
        // column tiles a wave, three or four waves and the ranges of k that come closest to one workgroup
        // a compute unit from below, all row blocks counted (measured at the Qwen3-8B sizes and 160 to 256
        // rows: 6,144 columns in 64 groups of three waves and 2 ranges, 4,096 in 32 groups of four waves
        // and 4 ranges; 7 to 18% faster than the kernel for any number of rows, which stays the faster one
        // for gated products and beyond 256 rows).
        int best = -1;
        for (int w = 4; w >= 3; --w) {
            const int groups = (n_tiles + 2 * w - 1) / (2 * w);
            const int r = max(1, min(min(units / max(groups * row_blocks, 1), k_steps / 2), 16));
            if (groups * r * row_blocks > best && groups * r * row_blocks <= units) {
                best = groups * r * row_blocks;
                *waves_a_group = w;
                *ranges = r;
            }
        }
        if (best < 0) {                       // more column groups than compute units: four waves, k whole
            *waves_a_group = 4;
            *ranges = 1;
        }
        *tiles_a_wave = 2;
        return;
    }
    auto ranges_for = [&](int groups) { return max(1, min(min(units / max(groups, 1), k_steps / 2), 16)); };
    int rt = mid_tiles_per_wave(N, gated), waves = 4;
    if (gated) {
        // a wave takes one pair of gate and up tiles; three to eight waves a workgroup, whichever
        // comes closest to 256 workgroups from below (24,576 columns: 256 workgroups of 3 waves,
        // 5% faster at 64 rows and 11% at 128 than 192 of 4; 34,816 columns: 218 of 5 waves, 12 to 17%
        // faster than 136 of 8); eight where even those are more than 256
        const int pairs = (n_tiles + 1) / 2;
        int best = 0;
        waves = 8;
        for (int w = 3; w <= 8; ++w) {
            const int groups = (pairs + w - 1) / w;
            if (groups <= units && groups > best) {
                best = groups;
                waves = w;
            }
        }
    }
    int groups = (n_tiles + waves * rt - 1) / (waves * rt);
    int splits = groups >= most ? 1 : ranges_for(groups);
    if (!gated && rt == 1 && groups * splits < most) {
        const int groups2 = (n_tiles + 7) / 8, splits2 = ranges_for(groups2);
        if (groups2 * splits2 > groups * splits) {
            rt = 2;
            splits = splits2;
        }
    }
    *tiles_a_wave = rt;
    *waves_a_group = waves;
    *ranges = splits;
}

// How many ranges of k a product of this shape is cut into (the caller sizes `part` by it).
extern "C" int tli_gemm_mid_splits(int N, int K, int gated) {
    int rt, waves, splits;
    mid_plan(N, K, gated, 1, &rt, &waves, &splits);
    return splits;
}

// The same for M rows (more than 128: row blocks side by side).
extern "C" int tli_gemm_mid_splits_rows(int M, int N, int K, int gated) {
    int rt, waves, splits;
    mid_plan(N, K, gated, (M + 127) / 128, &rt, &waves, &splits);
    return splits;
}

// y[M,N] = x[M,K] . W^T for 1 <= M <= 256 (a gated product: 128), W in the decode layout (`gated` as tiled = 2 of
// tli_gemm_skinny_bf16: y is [M, N/2] bfloat16).  `part`: splits*M*N floats when
// splits > 1 (splits as returned by tli_gemm_mid_splits, or forced by the caller); with
// y null the partial sums [splits][M][N] are left for the consumer to add (tli_gemm_mid_reduce,
// or tli_add_rmsnorm);
// cfg 0 picks the launch shape, else DEPTH*100 + RT*10 + WAVES.
extern "C" int tli_gemm_mid_bf16(const void* x, const void* w, void* y, float* part, int M, int N, int K,
                                 int y_dtype, int gated, int splits, int cfg, void* stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > MID_MAX_ROWS || (gated && M > 128))
        return tli_fail("gemm_mid: %d rows, at most %d (%d for a gated product)", M, MID_MAX_ROWS, 128);
    if (K <= 0 || K % 8) return tli_fail("gemm_mid: K = %d must be a positive multiple of 8", K);
    if (y_dtype != TLI_BF16 && y_dtype != TLI_F32) return tli_fail("gemm_mid: bad output dtype %d", y_dtype);
    if (gated && (N % 32 || y_dtype != TLI_BF16))
        return tli_fail("gemm_mid: a gated product needs N %% 32 == 0 and bfloat16 output");
    if (splits < 1 || splits > 64) return tli_fail("gemm_mid: %d splits", splits);
    if (splits > 1 && !part) return tli_fail("gemm_mid: splits need a buffer for partial sums");
    if (!y && (splits < 2 || gated)) return tli_fail("gemm_mid: only a plain product with split k can leave its partial sums");
    if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)part | (uintptr_t)y) & 15) return tli_fail("gemm_mid: operands must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    if (cfg == 0) {
        // more workgroups than compute units cost more than they bring (measured at the layer
        // sizes of Qwen3-14B and 32B): a gated product then takes eight waves a workgroup, a
        // plain one whose k ranges push it over takes two column tiles a wave
        int rt, planned, waves;
        mid_plan(N, K, gated, (M + 127) / 128, &rt, &waves, &planned);
        if (splits != planned && M <= 128) {                          // (ranges forced by the caller)
            rt = mid_tiles_per_wave(N, gated);
            const int groups = ((N + 15) / 16 + waves * rt - 1) / (waves * rt);
            if (!gated && rt == 1 && (long)groups * splits > tli_compute_units()) rt = 2;
        }
        cfg = 200 + 10 * rt + waves;
    }
    if (gated && (cfg / 10) % 10 < 2) return tli_fail("gemm_mid: a gated product needs pairs of row tiles");
#define MID_CASE(D, R, W) case D * 100 + R * 10 + W: return launch_mid<R, W, D>(xp, wp, y, part, M, N, K, y_dtype, gated, splits, s);
    switch (cfg) {
        MID_CASE(2, 1, 4) MID_CASE(3, 1, 4) MID_CASE(2, 1, 8) MID_CASE(4, 1, 8)
        MID_CASE(2, 2, 4) MID_CASE(4, 2, 4) MID_CASE(2, 2, 8)
        MID_CASE(2, 2, 3) MID_CASE(2, 2, 5) MID_CASE(2, 2, 6) MID_CASE(2, 2, 7)
        default: return tli_fail("gemm_mid: unknown configuration %d", cfg);
    }
}

// y[M,N] = sum over the partial products in `part` [splits][M][N], in split order.
extern "C" int tli_gemm_mid_reduce(const float* part, void* y, int M, int N, int splits, int y_dtype, void* stream) {
    if (M <= 0 || N <= 0) return 0;
    if (!part || !y || splits < 1) return tli_fail("gemm_mid_reduce: bad arguments");
    hipStream_t s = (hipStream_t)stream;
    if (y_dtype == TLI_BF16) launch_gemm_reduce(part, (bf16_t*)y, M, N, splits, 0, s);
    else if (y_dtype == TLI_F32) launch_gemm_reduce(part, (float*)y, M, N, splits, 0, s);
    else return tli_fail("gemm_mid_reduce: bad output dtype %d", y_dtype);
    return tli_check_launch("gemm_mid_reduce");
}
