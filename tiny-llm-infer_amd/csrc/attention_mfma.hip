// Attention over the paged cache on the matrix cores, bfloat16 storage,
// float32 scores, softmax and accumulation.  Two kernels share one tile routine:
//
//   decode:  every sequence brings one row.  A workgroup owns one (sequence, kv
//            head, key split); its four waves take the 32-key blocks of the
//            split in turn and are merged through LDS; splits are merged by a
//            second small kernel.
//   prefill: sequences bring portions of prompts (and single rows beside them).
//            A workgroup owns up to 4*RQ consecutive rows of one sequence and
//            one kv head; each wave owns RQ rows and walks the keys 0..p (or
//            the window) once.
//
// Same mathematics as the plain kernel (kernels/src/paged_attention_cpu.cpp:16-69):
// s_t = (q.k_t)*scale over the visible keys, softmax, weighted sum of values,
// kv head = head / (heads / kv_heads).
//
// Tile routine.  A wave holds 16 "columns": (query row, head of the kv group)
// pairs.  v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] B[32x16]; lane l holds
// A[l%16][8 k-slots of group c=l/16], B[those k-slots][l%16], D[4c..4c+3][l%16].
//   scores:  A = K tile (16 keys x head dims), B = Q^T  -> D[key][column]
//   output:  A = V^T tile (16 dims x 32 keys), B = P^T  -> D[dim][column]
// Keys are stored [slot][dim] and values transposed [dim][slot], so both A
// operands are 8- or 16-byte loads straight from the cache.  After the score
// MFMAs a lane holds, for its column, the keys 4c..4c+3 of two 16-key tiles:
// exactly the 8 k-slots of its group for the output MFMA, so probabilities
// never leave the lane's registers.  Softmax statistics are per column and
// thus per lane (replicated over the 4 lane groups).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

union Frag {
    uint4 u;
    uint2 h[2];
    bf16_t e[8];
    bf16x8 v;
};

struct CacheView {
    const bf16_t* k;          // [pages][kv_heads][page_size][head_dim]
    const bf16_t* v;          // [pages][kv_heads][head_dim][page_size]
    const int* table;         // this sequence's block table
    int table_width, page_size, page_shift, num_pages, kv_heads, head_dim, kv_head;

    // page of a key; -1 where the table holds none (or ends)
    __device__ __forceinline__ int page_of(int key) const {
        const int idx = key >> page_shift;
        return idx < table_width ? table[idx] : -1;
    }
};

// One wave's state for 16 columns.
template <int NJ, int ND>
struct Tile {
    Frag q[NJ];               // B operand of the score MFMAs: this lane's column, dims of group c
    f32x4 acc[ND];            // O^T[dim = 16*dt + 4c + i][column]
    float m, l;               // running maximum and sum of this lane's column
    int pos, lo;              // this column sees keys lo..pos (pos < lo: an idle column)
};

template <int NJ, int ND>
__device__ __forceinline__ void tile_init(Tile<NJ, ND>& t) {
#pragma unroll
    for (int d = 0; d < ND; ++d) t.acc[d] = (f32x4){0.f, 0.f, 0.f, 0.f};
    t.m = -INFINITY;
    t.l = 0.f;
}

// Load the query of this lane's column: dims [c*8*NJ + 8j, +8) for j < NJ.
template <int NJ, int ND>
__device__ __forceinline__ void tile_load_q(Tile<NJ, ND>& t, const bf16_t* q_head, int head_dim, bool live) {
    const int c = (threadIdx.x % 64) / 16;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int d = c * 8 * NJ + j * 8;
        t.q[j].u = (live && d < head_dim) ? *reinterpret_cast<const uint4*>(q_head + d) : make_uint4(0, 0, 0, 0);
    }
}

// Process the 32 keys t0 .. t0+31 (t0 a multiple of 32).
template <int NJ, int ND>
__device__ __forceinline__ void tile_step(Tile<NJ, ND>& t, const CacheView& cv, int t0, float scale) {
    const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
    // ---- scores: two 16-key tiles --------------------------------------
    f32x4 s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int key = t0 + u * 16 + r;                       // the key this lane loads as an A row
        const int page = cv.page_of(key);
        const bool ok = page >= 0 && page < cv.num_pages;
        const bf16_t* kp = cv.k + (((size_t)(ok ? page : 0) * cv.kv_heads + cv.kv_head) * cv.page_size +
                                   (key & (cv.page_size - 1))) * cv.head_dim;
        s[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int d = c * 8 * NJ + j * 8;
            Frag a;
            a.u = (ok && d < cv.head_dim) ? *reinterpret_cast<const uint4*>(kp + d) : make_uint4(0, 0, 0, 0);
            s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, t.q[j].v, s[u], 0, 0, 0);
        }
    }
    // ---- values: issue the loads before the softmax arithmetic ----------------
    // lane (dim r of tile dt, group c) takes keys t0+4c..+3 and t0+16+4c..+3
    Frag vt[ND];
    {
        const int key_a = t0 + 4 * c, key_b = t0 + 16 + 4 * c;
        const int page_a = cv.page_of(key_a), page_b = cv.page_of(key_b);
        const bool ok_a = page_a >= 0 && page_a < cv.num_pages, ok_b = page_b >= 0 && page_b < cv.num_pages;
        const size_t head_stride = (size_t)cv.head_dim * cv.page_size;
        const bf16_t* va = cv.v + ((size_t)(ok_a ? page_a : 0) * cv.kv_heads + cv.kv_head) * head_stride +
                           (key_a & (cv.page_size - 1));
        const bf16_t* vb = cv.v + ((size_t)(ok_b ? page_b : 0) * cv.kv_heads + cv.kv_head) * head_stride +
                           (key_b & (cv.page_size - 1));
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            const size_t off = (size_t)(dt * 16 + r) * cv.page_size;
            vt[dt].h[0] = ok_a ? *reinterpret_cast<const uint2*>(va + off) : make_uint2(0, 0);
            vt[dt].h[1] = ok_b ? *reinterpret_cast<const uint2*>(vb + off) : make_uint2(0, 0);
        }
    }
    // ---- softmax over this column -----------------------------------------
    float p[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = t0 + u * 16 + 4 * c + i;
            const bool seen = key >= t.lo && key <= t.pos;
            p[u][i] = seen ? s[u][i] * scale : -INFINITY;
            mx = fmaxf(mx, p[u][i]);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(t.m, mx);
    const float base = (m_new == -INFINITY) ? 0.f : m_new;      // nothing seen yet: all p become 0
    const float corr = __expf(t.m - base);                       // exp(-inf) = 0 on the first block
    Frag pb;
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bf16_t rounded = f32_to_bf16(__expf(p[u][i] - base));
            pb.e[u * 4 + i] = rounded;
            sum += bf16_to_f32(rounded);           // the sum uses what the matrix core will multiply
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    t.l = t.l * corr + sum;
    t.m = m_new;
    // ---- output --------------------------------------------------------------
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) t.acc[dt][i] *= corr;
        t.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt].v, pb.v, t.acc[dt], 0, 0, 0);
    }
}

// --------------------------------------------------------------------- decode --
// grid (splits, kv_heads * head_tiles, rows); 256 threads
template <int NJ, int ND>
__global__ void __launch_bounds__(256)
attention_decode_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out, float* __restrict__ partial,
                        const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                        const int* __restrict__ positions, const int* __restrict__ seq_of_row,
                        const int* __restrict__ tables, int table_width, int page_size, int page_shift,
                        int num_pages, int heads, int kv_heads, int head_dim, float scale, int window,
                        int splits, int keys_per_split) {
    extern __shared__ float lds[];       // 3 waves x 64 lanes x (ND*4 + 2)
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, r = lane % 16, c = lane / 16;
    const int split = blockIdx.x, row = blockIdx.z;
    const int group = heads / kv_heads;
    const int head_tiles = (group + 15) / 16;
    const int kv_head = blockIdx.y / head_tiles, head_tile = blockIdx.y % head_tiles;
    const int col_head = head_tile * 16 + r;                  // head inside the kv group
    const bool live = col_head < group;
    const int head = kv_head * group + col_head;
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;

    CacheView cv{k_cache, v_cache, tables + (size_t)seq_of_row[row] * table_width, table_width, page_size,
                 page_shift, num_pages, kv_heads, head_dim, kv_head};
    Tile<NJ, ND> t;
    tile_init(t);
    t.pos = live ? pos : -1;
    t.lo = live ? lo : 0;
    tile_load_q(t, q + ((size_t)row * heads + (live ? head : 0)) * head_dim, head_dim, live);

    // this split's keys, in 32-key blocks that the waves take in turn
    const int first_block = lo / 32;
    const int begin = first_block * 32 + split * keys_per_split;
    const int end = min(pos + 1, begin + keys_per_split);
    for (int t0 = begin + wave * 32; t0 < end; t0 += 4 * 32) tile_step(t, cv, t0, scale);

    // merge the four waves: waves 1..3 hand over (m, l, acc), wave 0 combines in wave order
    const int stride = ND * 4 + 2;
    if (wave > 0) {
        float* dst = lds + ((size_t)(wave - 1) * 64 + lane) * stride;
        dst[0] = t.m;
        dst[1] = t.l;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[2 + dt * 4 + i] = t.acc[dt][i];
    }
    __syncthreads();
    if (wave != 0) return;
    float m = t.m;
    for (int w = 0; w < 3; ++w) m = fmaxf(m, lds[((size_t)w * 64 + lane) * stride]);
    const float base = (m == -INFINITY) ? 0.f : m;
    float f = __expf(t.m - base);
    float l = t.l * f;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) t.acc[dt][i] *= f;
    for (int w = 0; w < 3; ++w) {
        const float* src = lds + ((size_t)w * 64 + lane) * stride;
        f = __expf(src[0] - base);
        l += src[1] * f;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) t.acc[dt][i] += src[2 + dt * 4 + i] * f;
    }
    if (!live) return;
    if (splits == 1) {
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* o = out + ((size_t)row * heads + head) * head_dim;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            uint2 packed;
            packed.x = (uint32_t)f32_to_bf16(t.acc[dt][0] * inv) | ((uint32_t)f32_to_bf16(t.acc[dt][1] * inv) << 16);
            packed.y = (uint32_t)f32_to_bf16(t.acc[dt][2] * inv) | ((uint32_t)f32_to_bf16(t.acc[dt][3] * inv) << 16);
            *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
        }
    } else {
        // partial[row][head][split][head_dim + 2]: unnormalised sum, then maximum and sum of weights
        float* dst = partial + (((size_t)row * heads + head) * splits + split) * (head_dim + 2);
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
            *reinterpret_cast<f32x4*>(dst + dt * 16 + 4 * c) = t.acc[dt];
        if (c == 0) {
            dst[head_dim] = m;
            dst[head_dim + 1] = l;
        }
    }
}

// grid (heads, rows); one thread per output element
__global__ void attention_merge_splits_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out,
                                              int heads, int head_dim, int splits) {
    const int head = blockIdx.x, row = blockIdx.y;
    const float* src = partial + ((size_t)row * heads + head) * splits * (head_dim + 2);
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, src[(size_t)s * (head_dim + 2) + head_dim]);
    const float base = (m == -INFINITY) ? 0.f : m;
    float l = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* p = src + (size_t)s * (head_dim + 2);
        l += p[head_dim + 1] * __expf(p[head_dim] - base);
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* p = src + (size_t)s * (head_dim + 2);
            a += p[d] * __expf(p[head_dim] - base);
        }
        out[((size_t)row * heads + head) * head_dim + d] = f32_to_bf16(a * inv);
    }
}

// -------------------------------------------------------------------- prefill --
// grid (row blocks upper bound, kv_heads * head_tiles); 256 threads.
// A wave owns `rq` consecutive rows of one sequence x min(group, 16) heads.
template <int NJ, int ND>
__global__ void __launch_bounds__(256)
attention_prefill_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                         const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                         const int* __restrict__ row_start, const int* __restrict__ seq_start,
                         int num_seqs, const int* __restrict__ tables, int table_width, int page_size,
                         int page_shift, int num_pages, int heads, int kv_heads, int head_dim,
                         float scale, int window, int rq) {
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, r = lane % 16, c = lane / 16;
    const int group = heads / kv_heads;
    const int head_tiles = (group + 15) / 16;
    const int kv_head = blockIdx.y / head_tiles, head_tile = blockIdx.y % head_tiles;
    const int heads_here = min(16, group - head_tile * 16);
    const int rows_per_block = 4 * rq;
    // which sequence and which of its row blocks is this workgroup's?
    int block = blockIdx.x, seq = 0, first_row = 0, n_rows = 0;
    for (; seq < num_seqs; ++seq) {
        first_row = row_start[seq];
        n_rows = row_start[seq + 1] - first_row;
        const int blocks = (n_rows + rows_per_block - 1) / rows_per_block;
        if (block < blocks) break;
        block -= blocks;
    }
    if (seq >= num_seqs) return;
    const int local0 = block * rows_per_block + wave * rq;    // this wave's first row in the sequence's portion
    if (local0 >= n_rows) return;
    const int my_rows = min(rq, n_rows - local0);
    // column r = (row r / heads_here, head r % heads_here)
    const int col_row = r / heads_here, col_head = head_tile * 16 + r % heads_here;
    const bool live = col_row < my_rows;
    const int row = first_row + local0 + (live ? col_row : 0);
    const int head = kv_head * group + col_head;
    const int pos = seq_start[seq] + local0 + col_row;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;

    CacheView cv{k_cache, v_cache, tables + (size_t)seq * table_width, table_width, page_size, page_shift,
                 num_pages, kv_heads, head_dim, kv_head};
    Tile<NJ, ND> t;
    tile_init(t);
    t.pos = live ? pos : -1;
    t.lo = live ? lo : 0;
    tile_load_q(t, q + ((size_t)row * heads + head) * head_dim, head_dim, live);

    const int first_pos = seq_start[seq] + local0, last_pos = first_pos + my_rows - 1;
    const int wave_lo = window > 0 ? max(0, first_pos - window + 1) : 0;
    for (int t0 = (wave_lo / 32) * 32; t0 <= last_pos; t0 += 32) tile_step(t, cv, t0, scale);

    if (!live) return;
    const float inv = t.l > 0.f ? 1.0f / t.l : 0.f;
    bf16_t* o = out + ((size_t)row * heads + head) * head_dim;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
        uint2 packed;
        packed.x = (uint32_t)f32_to_bf16(t.acc[dt][0] * inv) | ((uint32_t)f32_to_bf16(t.acc[dt][1] * inv) << 16);
        packed.y = (uint32_t)f32_to_bf16(t.acc[dt][2] * inv) | ((uint32_t)f32_to_bf16(t.acc[dt][3] * inv) << 16);
        *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
    }
}

// ------------------------------------------------------------------------ host --
static int log2_exact(int v) {
    int s = 0;
    while ((1 << s) < v) ++s;
    return (1 << s) == v ? s : -1;
}

static int check_common(const char* what, int heads, int kv_heads, int head_dim, int page_size,
                        int table_width, int num_pages) {
    if (head_dim < 16 || head_dim > 256 || head_dim % 16)
        return tli_fail("%s: head_dim %d must be a multiple of 16 from 16 to 256", what, head_dim);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
        return tli_fail("%s: heads %d must be a multiple of kv heads %d", what, heads, kv_heads);
    if (page_size < 4 || log2_exact(page_size) < 0)
        return tli_fail("%s: page size %d must be a power of two, at least 4", what, page_size);
    if (table_width <= 0 || num_pages <= 0) return tli_fail("%s: bad cache geometry", what);
    return 0;
}

#define DISPATCH_HEAD_DIM(CALL)                                   \
    switch (head_dim / 16) {                                      \
        case 1: CALL(1, 1); break;                                \
        case 2: CALL(1, 2); break;                                \
        case 3: CALL(2, 3); break;                                \
        case 4: CALL(2, 4); break;                                \
        case 5: CALL(3, 5); break;                                \
        case 6: CALL(3, 6); break;                                \
        case 7: CALL(4, 7); break;                                \
        case 8: CALL(4, 8); break;                                \
        case 9: CALL(5, 9); break;                                \
        case 10: CALL(5, 10); break;                              \
        case 11: CALL(6, 11); break;                              \
        case 12: CALL(6, 12); break;                              \
        case 13: CALL(7, 13); break;                              \
        case 14: CALL(7, 14); break;                              \
        case 15: CALL(8, 15); break;                              \
        default: CALL(8, 16); break;                              \
    }

// Every row is its sequence's only row in this step.  `partial` holds
// rows*heads*splits*(head_dim+2) floats when splits > 1.
extern "C" int tli_attention_decode_bf16(
    const void* q, void* out, float* partial, const void* k_cache, const void* v_cache,
    const int* positions, const int* seq_of_row, const int* tables, int table_width, int page_size,
    int num_pages, int rows, int heads, int kv_heads, int head_dim, float scale, int window,
    int splits, int keys_per_split, void* stream) {
    if (rows <= 0) return 0;
    if (check_common("attention_decode", heads, kv_heads, head_dim, page_size, table_width, num_pages)) return 1;
    if (splits < 1 || splits > 65535 || keys_per_split <= 0 || keys_per_split % 128)
        return tli_fail("attention_decode: %d splits of %d keys (keys per split must be a multiple of 128)",
                        splits, keys_per_split);
    if (splits > 1 && !partial) return tli_fail("attention_decode: splits need a partial buffer");
    if (rows > 65535) return tli_fail("attention_decode: %d rows exceed the grid limit", rows);
    hipStream_t s = (hipStream_t)stream;
    const int group = heads / kv_heads, head_tiles = (group + 15) / 16;
    dim3 grid(splits, kv_heads * head_tiles, rows);
    const int shift = log2_exact(page_size);
#define CALL(NJ, ND)                                                                                    \
    attention_decode_kernel<NJ, ND><<<grid, 256, 3 * 64 * (ND * 4 + 2) * sizeof(float), s>>>(           \
        (const bf16_t*)q, (bf16_t*)out, partial, (const bf16_t*)k_cache, (const bf16_t*)v_cache,        \
        positions, seq_of_row, tables, table_width, page_size, shift, num_pages, heads, kv_heads,       \
        head_dim, scale, window, splits, keys_per_split)
    DISPATCH_HEAD_DIM(CALL)
#undef CALL
    if (tli_check_launch("attention_decode")) return 1;
    if (splits > 1) {
        attention_merge_splits_kernel<<<dim3(heads, rows), 64, 0, s>>>(partial, (bf16_t*)out, heads, head_dim, splits);
        return tli_check_launch("attention_merge_splits");
    }
    return 0;
}

// Rows of a sequence are contiguous and ascend in position; row_start has num_seqs+1 entries.
extern "C" int tli_attention_prefill_bf16(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* row_start,
    const int* seq_start, int num_seqs, int rows, const int* tables, int table_width, int page_size,
    int num_pages, int heads, int kv_heads, int head_dim, float scale, int window, void* stream) {
    if (rows <= 0 || num_seqs <= 0) return 0;
    if (check_common("attention_prefill", heads, kv_heads, head_dim, page_size, table_width, num_pages)) return 1;
    hipStream_t s = (hipStream_t)stream;
    const int group = heads / kv_heads, head_tiles = (group + 15) / 16;
    const int rq = group >= 16 ? 1 : 16 / group;
    const int rows_per_block = 4 * rq;
    const long blocks = (rows + rows_per_block - 1) / rows_per_block + num_seqs;   // upper bound
    if (blocks > 2147483647L) return tli_fail("attention_prefill: too many rows");
    dim3 grid((unsigned)blocks, kv_heads * head_tiles);
    const int shift = log2_exact(page_size);
#define CALL(NJ, ND)                                                                                  \
    attention_prefill_kernel<NJ, ND><<<grid, 256, 0, s>>>(                                            \
        (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache, row_start,    \
        seq_start, num_seqs, tables, table_width, page_size, shift, num_pages, heads, kv_heads,       \
        head_dim, scale, window, rq)
    DISPATCH_HEAD_DIM(CALL)
#undef CALL
    return tli_check_launch("attention_prefill");
}
