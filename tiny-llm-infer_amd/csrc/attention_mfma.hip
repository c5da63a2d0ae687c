// Attention over the paged cache on the matrix cores, bfloat16 storage,
// float32 scores, softmax and accumulation.  Two kernels share one tile routine:
//
//   decode:  every sequence brings one row.  A workgroup owns one (sequence, kv
//            head, key split); its four waves take the 32-key blocks of the
//            split in turn, each asking for its next block before it multiplies
//            the current one, and are merged through LDS; splits are merged by a
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
#include <type_traits>

#pragma clang diagnostic ignored "-Winline-asm"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;       // 16 bytes in flight, as a first-class vector

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
    f32x4 ls;                 // the column's sum of weights, four times (a row of ones times P^T),
    float l;                  // or summed by the lanes: one of the two is used, the other stays 0
    float m, nb;              // base of the column's exponentials, -inf while nothing is seen; -base (0 then)
    int pos, lo;              // this column sees keys lo..pos (pos < lo: an idle column)
};

template <int NJ, int ND>
__device__ __forceinline__ void tile_init(Tile<NJ, ND>& t) {
#pragma unroll
    for (int d = 0; d < ND; ++d) t.acc[d] = (f32x4){0.f, 0.f, 0.f, 0.f};
    t.ls = (f32x4){0.f, 0.f, 0.f, 0.f};
    t.l = 0.f;
    t.m = -INFINITY;
    t.nb = 0.f;
}

// The sum of the weights of this lane's column.
template <int NJ, int ND>
__device__ __forceinline__ float tile_sum(const Tile<NJ, ND>& t) { return t.ls[0] + t.l; }

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

// Scores, softmax update and output accumulation of CT column tiles for 32 keys whose
// fragments they share.  Row 4c+i of score tile u (and k-slot 4u+i of lane group c in the
// output MFMA) is the key  key_c0 + u*u_stride + i.
//
// A weight is exp2(score * scale*log2(e) - base): one fused multiply-add and one
// v_exp_f32.  The base of a column follows the column's maximum lazily: it stays as
// long as no score of the wave lies more than 2^LAZY_BITS above its column's base, which
// bounds the weights by 2^LAZY_BITS instead of 1 (harmless in float32 sums and in
// bfloat16 weights).  Whether it may stay is decided from each lane's own 8 scores, so
// the usual round needs no exchange between lanes at all: only when a base has to move
// are the columns' maxima gathered over the four lane groups and the accumulators
// rescaled.  MFMA_SUM: the sum of a column's weights is one more output MFMA, with a row
// of ones for the values (it adds the weights as rounded to bfloat16, the ones that the
// values meet); else the lanes add them (the decode kernel, which is short of registers
// and not of vector arithmetic).
// MASK = false skips the comparison with lo..pos when the caller knows every key is
// seen by every live column (an idle column then computes on zeros; it is never stored).
// The phases (all score MFMAs, all softmax arithmetic, all output MFMAs) let one tile's
// vector arithmetic run beside another tile's matrix instructions.
#define LAZY_BITS 8.0f
template <int NJ, int ND, int CT, bool MASK, bool MFMA_SUM = true>
__device__ __forceinline__ void tiles_consume(Tile<NJ, ND> (&tiles)[CT], const Frag (&ka)[2][NJ],
                                              const Frag (&vt)[ND], int key_c0, int u_stride,
                                              float scale_log2) {
    f32x4 s[CT][2];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            s[ct][u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                s[ct][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[u][j].v, tiles[ct].q[j].v, s[ct][u], 0, 0, 0);
        }
    // this lane's maxima, and whether some base has to move
    float mx[CT];
    bool move = false;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        Tile<NJ, ND>& t = tiles[ct];
        mx[ct] = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (MASK) {
                    const int key = key_c0 + u * u_stride + i;
                    s[ct][u][i] = (key >= t.lo && key <= t.pos) ? s[ct][u][i] : -INFINITY;
                }
                mx[ct] = fmaxf(mx[ct], s[ct][u][i]);
            }
        // (nothing seen before and nothing now: -inf + inf is NaN and compares false)
        move = move || fmaf(mx[ct], scale_log2, -t.m) > LAZY_BITS;
    }
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            Tile<NJ, ND>& t = tiles[ct];
            const float m_new = fmaxf(t.m, quad_rows_max(mx[ct]) * scale_log2);
            const float base = (m_new == -INFINITY) ? 0.f : m_new;
            const float corr = __builtin_amdgcn_exp2f(t.m - base);       // exp2(-inf) = 0 the first time
            t.m = m_new;
            t.nb = -base;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) t.acc[dt][i] *= corr;
            if (MFMA_SUM) {
#pragma unroll
                for (int i = 0; i < 4; ++i) t.ls[i] *= corr;
            } else {
                t.l *= corr;
            }
        }
    }
    Frag pb[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const float nb = tiles[ct].nb;
        float p[2][4];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) p[u][i] = __builtin_amdgcn_exp2f(fmaf(s[ct][u][i], scale_log2, nb));
        pb[ct].u = make_uint4(pack_bf16x2(p[0][0], p[0][1]), pack_bf16x2(p[0][2], p[0][3]),
                              pack_bf16x2(p[1][0], p[1][1]), pack_bf16x2(p[1][2], p[1][3]));
        if (!MFMA_SUM) {
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) sum += p[u][i];
            tiles[ct].l += quad_rows_sum(sum);
        }
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
            tiles[ct].acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt].v, pb[ct].v, tiles[ct].acc[dt], 0, 0, 0);
    if (MFMA_SUM) {
        Frag ones;
        ones.u = make_uint4(0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
            tiles[ct].ls = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pb[ct].v, tiles[ct].ls, 0, 0, 0);
    }
}

// The same for one tile, the lanes adding the weights.
template <int NJ, int ND, bool MASK>
__device__ __forceinline__ void tile_consume(Tile<NJ, ND>& t, const Frag (&ka)[2][NJ], const Frag (&vt)[ND],
                                             int key_c0, int u_stride, float scale_log2) {
    Tile<NJ, ND> (&one)[1] = reinterpret_cast<Tile<NJ, ND>(&)[1]>(t);
    tiles_consume<NJ, ND, 1, MASK, false>(one, ka, vt, key_c0, u_stride, scale_log2);
}

// The phases of tiles_consume as functions of their own, for a caller that overlaps them: the
// score MFMAs of the next 32 keys run beside the vector arithmetic of these.
template <int NJ, int ND, int CT>
__device__ __forceinline__ void tiles_scores(const Tile<NJ, ND> (&tiles)[CT], const Frag (&ka)[2][NJ], f32x4 (&s)[CT][2]) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int u = 0; u < 2; ++u) s[ct][u] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // (the 2 CT sums take turns, so that no MFMA waits for the one before it)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int u = 0; u < 2; ++u)
                s[ct][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[u][j].v, tiles[ct].q[j].v, s[ct][u], 0, 0, 0);
}

// Scores -> exponents of the weights, score * scale - base, in place; the bases move (and the
// sums are rescaled) where an exponent would pass LAZY_BITS.  The maxima are taken of the
// exponents, the results of a multiply-add, not of the MFMA's output, which the compiler would
// first pass through a second instruction that quiets signalling NaNs.
template <int NJ, int ND, int CT, bool MASK>
__device__ __forceinline__ void tiles_exponents(Tile<NJ, ND> (&tiles)[CT], f32x4 (&s)[CT][2], int key_c0, int u_stride,
                                                float scale_log2) {
    float top[CT];
    bool move = false;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        Tile<NJ, ND>& t = tiles[ct];
        top[ct] = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (MASK) {
                    const int key = key_c0 + u * u_stride + i;
                    s[ct][u][i] = (key >= t.lo && key <= t.pos) ? s[ct][u][i] : -INFINITY;
                }
                s[ct][u][i] = fmaf(s[ct][u][i], scale_log2, t.nb);
                top[ct] = fmaxf(top[ct], s[ct][u][i]);
            }
        // (nothing seen before: the base is -inf and nb is 0, so the first key that is seen moves the
        // base; nothing seen now either: -inf > -inf is false)
        move = move || top[ct] > (t.m == -INFINITY ? -INFINITY : LAZY_BITS);
    }
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            Tile<NJ, ND>& t = tiles[ct];
            // top is relative to the old base (-nb, 0 while nothing was seen)
            const float m_new = fmaxf(t.m, quad_rows_max(top[ct]) - t.nb);
            const float base = (m_new == -INFINITY) ? 0.f : m_new;
            const float corr = __builtin_amdgcn_exp2f(t.m - base);       // exp2(-inf) = 0 the first time
            const float shift = -base - t.nb;                            // the exponents follow the base
            t.m = m_new;
            t.nb = -base;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) t.acc[dt][i] *= corr;
#pragma unroll
            for (int i = 0; i < 4; ++i) t.ls[i] *= corr;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) s[ct][u][i] += shift;
        }
    }
}

// Exponents -> weights, as the B operands of the output MFMAs.
template <int CT>
__device__ __forceinline__ void tiles_pack(const f32x4 (&s)[CT][2], Frag (&pb)[CT]) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        float p[2][4];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) p[u][i] = __builtin_amdgcn_exp2f(s[ct][u][i]);
        pb[ct].u = make_uint4(pack_bf16x2(p[0][0], p[0][1]), pack_bf16x2(p[0][2], p[0][3]),
                              pack_bf16x2(p[1][0], p[1][1]), pack_bf16x2(p[1][2], p[1][3]));
    }
}

// The weighted sums of the values, and the sums of the weights (a row of ones for the values).
template <int NJ, int ND, int CT>
__device__ __forceinline__ void tiles_output(Tile<NJ, ND> (&tiles)[CT], const Frag (&vt)[ND], const Frag (&pb)[CT]) {
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
            tiles[ct].acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt].v, pb[ct].v, tiles[ct].acc[dt], 0, 0, 0);
    Frag ones;
    ones.u = make_uint4(0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
        tiles[ct].ls = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pb[ct].v, tiles[ct].ls, 0, 0, 0);
}

// Process the 32 keys t0 .. t0+31 (t0 a multiple of 32) for CT column tiles that
// share the key and value fragments (one load from the cache, CT times the MFMAs).
template <int NJ, int ND, int CT>
__device__ __forceinline__ void tiles_step(Tile<NJ, ND> (&tiles)[CT], const CacheView& cv, int t0, float scale) {
    const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
    // ---- key fragments: two 16-key tiles -----------------------------------
    Frag ka[2][NJ];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int key = t0 + u * 16 + r;                       // the key this lane loads as an A row
        const int page = cv.page_of(key);
        const bool ok = page >= 0 && page < cv.num_pages;
        const bf16_t* kp = cv.k + (((size_t)(ok ? page : 0) * cv.kv_heads + cv.kv_head) * cv.page_size +
                                   (key & (cv.page_size - 1))) * cv.head_dim;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int d = c * 8 * NJ + j * 8;
            ka[u][j].u = (ok && d < cv.head_dim) ? *reinterpret_cast<const uint4*>(kp + d) : make_uint4(0, 0, 0, 0);
        }
    }
    // ---- value fragments: issued before the softmax arithmetic ------------------
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
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) tile_consume<NJ, ND, true>(tiles[ct], ka, vt, t0 + 4 * c, 16, scale);
}

template <int NJ, int ND>
__device__ __forceinline__ void tile_step(Tile<NJ, ND>& t, const CacheView& cv, int t0, float scale) {
    Tile<NJ, ND> (&one)[1] = reinterpret_cast<Tile<NJ, ND>(&)[1]>(t);
    tiles_step<NJ, ND, 1>(one, cv, t0, scale);
}

// --------------------------------------------------------------------- decode --
// The fragments of one block of 32 keys, as tile_consume takes them.
template <int NJ, int ND>
struct KeyBlock {
    Frag ka[2][NJ];
    Frag vt[ND];
};

// Ask for the 32 keys t0 .. t0+31.  Row 4c'+i of score tile u is the key t0 + 8c' + 4u + i
// (tile_consume is told so: key_c0 = t0 + 8c, u_stride = 4): the eight keys that a lane group
// multiplies the values of are then consecutive, and a lane takes them from the transposed
// values in one 16-byte load; both key rows of a lane (tile 0 and 1, four keys apart) and all
// its values lie in one page each, which holds at least 8 keys.  `seg` holds the block table
// entries seg_first .. seg_first+seg_len-1 in LDS.  No load is predicated, so that the
// fragments of the next block can be in flight while this one is multiplied (after a branch
// that may have issued loads the compiler waits for all loads in flight): a key without a page
// reads page 0 instead.  Such keys lie outside lo..pos, their scores are masked, and their
// values meet a weight of exactly 0; the cache is allocated zeroed, so they are finite.
template <int NJ, int ND>
__device__ __forceinline__ void decode_fetch(KeyBlock<NJ, ND>& b, const CacheView& cv, const int* seg,
                                             int seg_first, int seg_len, int t0) {
    const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
    auto page_at = [&](int key) {
        const int rel = (key >> cv.page_shift) - seg_first;          // >= 0: t0 is not before the split
        const int page = seg[min(rel, seg_len - 1)];
        return (unsigned)page < (unsigned)cv.num_pages ? page : 0;
    };
    const int in_page = cv.page_size - 1;
    const int key_k = t0 + 8 * (r / 4) + (r % 4);                    // tile 0; tile 1 is four keys on
    const bf16_t* kp = cv.k + (((size_t)page_at(key_k) * cv.kv_heads + cv.kv_head) * cv.page_size +
                               (key_k & in_page)) * cv.head_dim;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int d = c * 8 * NJ + j * 8;                        // past head_dim the query is zero
            b.ka[u][j].u = *reinterpret_cast<const uint4*>(kp + (size_t)u * 4 * cv.head_dim + (d < cv.head_dim ? d : 0));
        }
    const int key_v = t0 + 8 * c;
    const bf16_t* vp = cv.v + ((size_t)page_at(key_v) * cv.kv_heads + cv.kv_head) * ((size_t)cv.head_dim * cv.page_size) +
                       (key_v & in_page);
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
        b.vt[dt].u = *reinterpret_cast<const uint4*>(vp + (size_t)(dt * 16 + r) * cv.page_size);
}

// The step's raw projections [rows][(heads + 2 kv_heads) * head_dim] and what turns them
// into queries and keys, for the decode kernel that does that work itself
// (model/src/qwen3_paged_batch.cpp:180-236: per-head norm, rotation, cache write).
struct RawQkv {
    const bf16_t* qkv;
    const float* q_norm_w;    // [head_dim] or null
    const float* k_norm_w;
    const float* cos;         // [positions][head_dim / 2] or null
    const float* sin;
    float q_eps, k_eps;
    int write_cache;          // 0: the layer reads a cache that another layer writes
    // the decode kernel only: the projections as float32 partial sums [parts][rows][columns]
    // of a product whose k range was split (qkv is then not read); an element is their sum
    // in part order, rounded to bfloat16 as the product's own reduction would have
    const float* partial_sums;
    int parts;
    size_t part_stride;
};

// One head of the raw projections as a B operand of the score MFMAs (this lane: dims
// [c*8*NJ, +8*NJ) of the head at `src`), after the per-head RMS norm (if nw) and the
// half-split rotation (if cos_row).  head_dim == 32*NJ, so the first half of the head
// lies in lane groups 0 and 1 and the rotation partner of a lane is lane ^ 32.
// With psrc the head is taken from `parts` planes of float32 partial sums instead (the
// head's first element in plane 0 at psrc, planes part_stride floats apart).
template <int NJ>
__device__ __forceinline__ void head_from_raw(Frag (&out)[NJ], const bf16_t* src, const float* nw, float eps,
                                              const float* cos_row, const float* sin_row,
                                              const float* psrc = nullptr, int parts = 0, size_t part_stride = 0) {
    const int c = (threadIdx.x % 64) / 16;
    const int d0 = c * 8 * NJ;
    float x[NJ][8];
    if (psrc) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[j][e] = 0.f;
        // two planes a round, both asked for before either is added (the second of an odd
        // last round is the first again, and counts as zero)
        for (int p = 0; p < parts; p += 2) {
            const bool pair = p + 1 < parts;
            const float* from0 = psrc + (size_t)p * part_stride + d0;
            const float* from1 = psrc + (size_t)(pair ? p + 1 : p) * part_stride + d0;
            f32x4 v0[NJ][2], v1[NJ][2];
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                v0[j][0] = *reinterpret_cast<const f32x4*>(from0 + j * 8);
                v0[j][1] = *reinterpret_cast<const f32x4*>(from0 + j * 8 + 4);
                v1[j][0] = *reinterpret_cast<const f32x4*>(from1 + j * 8);
                v1[j][1] = *reinterpret_cast<const f32x4*>(from1 + j * 8 + 4);
            }
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[j][e] += v0[j][e / 4][e % 4];
                    x[j][e] += pair ? v1[j][e / 4][e % 4] : 0.f;
                }
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[j][e] = bf16_to_f32(f32_to_bf16(x[j][e]));
    } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            Frag f;
            f.u = *reinterpret_cast<const uint4*>(src + d0 + j * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[j][e] = bf16_to_f32(f.e[e]);
        }
    }
    if (nw) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += x[j][e] * x[j][e];
        ss = quad_rows_sum(ss);
        const float scale = 1.0f / sqrtf(ss / (float)(32 * NJ) + eps);
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[j][e] = nw[d0 + j * 8 + e] * x[j][e] * scale;
    }
    if (cos_row) {
        const int i0 = (c & 1) * 8 * NJ;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float partner = __shfl_xor(x[j][e], 32, 64);
                const float cs = cos_row[i0 + j * 8 + e], sn = sin_row[i0 + j * 8 + e];
                x[j][e] = c < 2 ? rotate_first_half(x[j][e], partner, cs, sn) : rotate_second_half(x[j][e], partner, cs, sn);
            }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        out[j].u = make_uint4(pack_bf16x2(x[j][0], x[j][1]), pack_bf16x2(x[j][2], x[j][3]),
                              pack_bf16x2(x[j][4], x[j][5]), pack_bf16x2(x[j][6], x[j][7]));
}

// The decode kernel's prologue shares the work on a head out over the four waves by slices of 8
// dims a lane (slice j of a lane: dims c*8*NJ + 8j ..): a wave fetches its slices, the waves
// exchange their parts of the sum of squares through LDS, and each finishes its slices.
// Eight elements of a head at `src` (bfloat16), or, with psrc, their sums over `parts` planes of
// float32 partial sums in part order (two planes a round, both asked for before either is
// added), rounded to bfloat16 as the product's own reduction would have.
__device__ __forceinline__ void slice_fetch(float (&x)[8], const bf16_t* src, const float* psrc, int parts,
                                            size_t part_stride) {
    if (psrc) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = 0.f;
        for (int p = 0; p < parts; p += 2) {
            const bool pair = p + 1 < parts;
            const float* from0 = psrc + (size_t)p * part_stride;
            const float* from1 = psrc + (size_t)(pair ? p + 1 : p) * part_stride;
            const f32x4 a0 = *reinterpret_cast<const f32x4*>(from0), a1 = *reinterpret_cast<const f32x4*>(from0 + 4);
            const f32x4 b0 = *reinterpret_cast<const f32x4*>(from1), b1 = *reinterpret_cast<const f32x4*>(from1 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[e] += a0[e];
                x[e] += pair ? b0[e] : 0.f;
                x[4 + e] += a1[e];
                x[4 + e] += pair ? b1[e] : 0.f;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = bf16_to_f32(f32_to_bf16(x[e]));
    } else {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(src);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = bf16_to_f32(f.e[e]);
    }
}

// Eight floats at p (16-byte aligned), or zeros for a null p.
__device__ __forceinline__ void load8(float (&v)[8], const float* p) {
    if (p) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[e] = a[e];
            v[4 + e] = b[e];
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
    }
}

// A slice after the norm (if normed: factor `scale`, weights nw8) and the half-split rotation
// (if rotate: cos8, sin8 of the slice's dims), as the score MFMAs take it.  The rotation partner
// of a lane is lane ^ 32 (head_dim == 32*NJ: the first half of the head lies in lane groups 0, 1).
__device__ __forceinline__ uint4 slice_finish(float (&x)[8], bool normed, const float (&nw8)[8], float scale,
                                              bool rotate, const float (&cos8)[8], const float (&sin8)[8]) {
    const int c = (threadIdx.x % 64) / 16;
    if (normed) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = nw8[e] * x[e] * scale;
    }
    if (rotate) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float partner = __shfl_xor(x[e], 32, 64);
            const float cs = cos8[e], sn = sin8[e];
            x[e] = c < 2 ? rotate_first_half(x[e], partner, cs, sn) : rotate_second_half(x[e], partner, cs, sn);
        }
    }
    return make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]), pack_bf16x2(x[6], x[7]));
}

// grid (kv_heads * head_tiles, rows, splits); 256 threads.  (Workgroups go to the eight dies in turn,
// in the order of the grid with x fastest: with the splits in x, split s of every row would run on the
// dies s, s + splits, .., and the dies of a row's last splits, which are short or empty, would idle
// while the others walk the whole ones.)  FUSED: queries come from the
// raw projections `raw` (q is not read), and the workgroup whose keys include the row's
// own position writes that key and value into the cache first; needs head_dim == 32*NJ
// and at most 16 heads a kv head (one workgroup per kv head and split).
template <int NJ, int ND, bool FUSED>
__global__ void __launch_bounds__(256, ND <= 8 ? 2 : 1)
attention_decode_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out, float* __restrict__ partial,
                        bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                        const int* __restrict__ positions, const int* __restrict__ seq_of_row,
                        const int* __restrict__ tables, int table_width, int page_size, int page_shift,
                        int num_pages, int heads, int kv_heads, int head_dim, float scale, int window,
                        int splits, int keys_per_split, RawQkv raw) {
    extern __shared__ float lds[];       // 4 waves x 64 lanes x (ND*4 + 2), then this split's table entries, FUSED: the prologue's sums of squares and slices of q
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, r = lane % 16, c = lane / 16;
    const int split = blockIdx.z, row = blockIdx.y;
    const int group = heads / kv_heads;
    const int head_tiles = (group + 15) / 16;
    const int kv_head = blockIdx.x / head_tiles, head_tile = blockIdx.x % head_tiles;
    const int col_head = head_tile * 16 + r;                  // head inside the kv group
    const bool live = col_head < group;
    const int head = kv_head * group + col_head;
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int* table = tables + (size_t)seq_of_row[row] * table_width;

    CacheView cv{k_cache, v_cache, table, table_width, page_size, page_shift, num_pages, kv_heads, head_dim,
                 kv_head};
    Tile<NJ, ND> t;
    tile_init(t);
    t.pos = live ? pos : -1;
    t.lo = live ? lo : 0;
    // this split's keys, in 32-key blocks that the waves take in turn
    const int first_block = lo / 32;
    const int begin = first_block * 32 + split * keys_per_split;
    const int end = min(pos + 1, begin + keys_per_split);
    // its part of the block table goes to LDS once, so that a block's addresses do not
    // wait for a table entry from memory first
    int* seg = reinterpret_cast<int*>(lds + 4 * 64 * (ND * 4 + 2));
    const int seg_first = begin >> page_shift;
    const int seg_len = begin < end ? ((end - 1) >> page_shift) - seg_first + 1 : 0;
    if (FUSED) {
        // The prologue (see slice_fetch): wave w has the slices j = w, w + 4, .. of the lane's query
        // head and, where this workgroup writes the row's own key, of the key head.
        constexpr int SJ = (NJ + 3) / 4;                  // slices a wave at most
        float* ssq = reinterpret_cast<float*>(seg + (((keys_per_split >> page_shift) + 2 + 3) & ~3));   // [q, k][wave][16]
        uint4* q_slices = reinterpret_cast<uint4*>(ssq + 2 * 4 * 16);                                   // [NJ][64]
        const size_t width = (size_t)(heads + 2 * kv_heads) * head_dim;
        const bf16_t* raw_row = raw.qkv + (size_t)row * width;
        const float* sums_row = raw.partial_sums ? raw.partial_sums + (size_t)row * width : nullptr;
        const bool own = raw.write_cache && begin <= pos && pos < end;       // the row's own key and value are this workgroup's
        // (an idle column computes on head 0; it is masked by its pos of -1)
        const size_t q_off = (size_t)(live ? head : 0) * head_dim + c * 8 * NJ;
        const size_t k_off = (size_t)(heads + kv_head) * head_dim + c * 8 * NJ;
        float xq[SJ][8], xk[SJ][8];
        // (the constants of a slice's norm and rotation are asked for with the slice, before the barrier)
        float nq[SJ][8], nk[SJ][8], cs[SJ][8], sn[SJ][8];
        const float* rot_at = raw.cos ? raw.cos + (size_t)pos * (head_dim / 2) + (c & 1) * 8 * NJ : nullptr;
        const float* rot_sin = raw.cos ? raw.sin + (size_t)pos * (head_dim / 2) + (c & 1) * 8 * NJ : nullptr;
        float sq = 0.f, sk = 0.f;
#pragma unroll
        for (int jj = 0; jj < SJ; ++jj) {
            const int j = jj * 4 + wave;
            if (j < NJ) {
                load8(cs[jj], rot_at ? rot_at + j * 8 : nullptr);
                load8(sn[jj], rot_sin ? rot_sin + j * 8 : nullptr);
                load8(nq[jj], raw.q_norm_w ? raw.q_norm_w + c * 8 * NJ + j * 8 : nullptr);
                load8(nk[jj], raw.k_norm_w ? raw.k_norm_w + c * 8 * NJ + j * 8 : nullptr);
                slice_fetch(xq[jj], raw_row + q_off + j * 8, sums_row ? sums_row + q_off + j * 8 : nullptr, raw.parts,
                            raw.part_stride);
#pragma unroll
                for (int e = 0; e < 8; ++e) sq += xq[jj][e] * xq[jj][e];
                if (own) {
                    slice_fetch(xk[jj], raw_row + k_off + j * 8, sums_row ? sums_row + k_off + j * 8 : nullptr, raw.parts,
                                raw.part_stride);
#pragma unroll
                    for (int e = 0; e < 8; ++e) sk += xk[jj][e] * xk[jj][e];
                }
            }
        }
        sq = quad_rows_sum(sq);
        sk = quad_rows_sum(sk);
        if (c == 0) {
            ssq[wave * 16 + r] = sq;
            ssq[(4 + wave) * 16 + r] = sk;
        }
        for (int i = threadIdx.x; i < seg_len; i += 256)
            seg[i] = seg_first + i < table_width ? table[seg_first + i] : -1;
        __syncthreads();
        const float q_ss = ssq[r] + ssq[16 + r] + ssq[32 + r] + ssq[48 + r];
        const float k_ss = ssq[64 + r] + ssq[80 + r] + ssq[96 + r] + ssq[112 + r];
        const float q_scale = 1.0f / sqrtf(q_ss / (float)(32 * NJ) + raw.q_eps);
        const float k_scale = 1.0f / sqrtf(k_ss / (float)(32 * NJ) + raw.k_eps);
        int own_page = -1;
        const int slot = pos & (page_size - 1);
        if (own) own_page = seg[(pos >> page_shift) - seg_first];
        const bool store = own && (unsigned)own_page < (unsigned)num_pages;
#pragma unroll
        for (int jj = 0; jj < SJ; ++jj) {
            const int j = jj * 4 + wave;
            if (j < NJ) {
                q_slices[j * 64 + lane] = slice_finish(xq[jj], raw.q_norm_w != nullptr, nq[jj], q_scale,
                                                       raw.cos != nullptr, cs[jj], sn[jj]);
                if (own) {
                    const uint4 kf = slice_finish(xk[jj], raw.k_norm_w != nullptr, nk[jj], k_scale,
                                                  raw.cos != nullptr, cs[jj], sn[jj]);
                    if (store && r == 0)
                        *reinterpret_cast<uint4*>(k_cache + (((size_t)own_page * kv_heads + kv_head) * page_size + slot) * head_dim +
                                                  c * 8 * NJ + j * 8) = kf;
                }
            }
        }
        if (store && wave == 3) {
            // the value: two elements a lane
            const bf16_t* src = raw_row + (size_t)(heads + kv_heads + kv_head) * head_dim;
            bf16_t* dst = v_cache + ((size_t)own_page * kv_heads + kv_head) * head_dim * page_size + slot;
            if (sums_row) {
                const float* from = sums_row + (size_t)(heads + kv_heads + kv_head) * head_dim;
                for (int d = lane; d < head_dim; d += 64) {
                    float v = 0.f;
                    for (int p = 0; p < raw.parts; p += 2) {
                        const bool pair = p + 1 < raw.parts;
                        const float a = from[(size_t)p * raw.part_stride + d];
                        const float b = from[(size_t)(pair ? p + 1 : p) * raw.part_stride + d];
                        v += a;
                        v += pair ? b : 0.f;
                    }
                    dst[(size_t)d * page_size] = cache_value(f32_to_bf16(v));
                }
            } else {
                for (int d = lane; d < head_dim; d += 64) dst[(size_t)d * page_size] = cache_value(src[d]);
            }
        }
        __syncthreads();           // the slices of q are in LDS, the row's own key and value in the cache
#pragma unroll
        for (int j = 0; j < NJ; ++j) t.q[j].u = q_slices[j * 64 + lane];
    } else {
        tile_load_q(t, q + ((size_t)row * heads + (live ? head : 0)) * head_dim, head_dim, live);
        for (int i = threadIdx.x; i < seg_len; i += 256)
            seg[i] = seg_first + i < table_width ? table[seg_first + i] : -1;
        __syncthreads();
    }

    // a wave's blocks are 128 keys apart; the next block is asked for before this one is
    // multiplied, two sets of registers taking turns.  Nothing is asked for twice and no load
    // of the loop is under a branch: the blocks are dealt to the two sets from the end, so that
    // the last block always comes into the first set and is multiplied after the loop; a wave
    // with an even number of blocks begins with one block in the second set.  (Asking for the
    // last block once more instead, as a loop without this must, was a tenth of the kernel's
    // time at the few hundred keys of a short context, where most waves have one block or two.)
    int t0 = begin + wave * 32;
    if (t0 < end) {
        const int last = t0 + (end - 1 - t0) / 128 * 128;
        KeyBlock<NJ, ND> b0, b1;
        if (((last - t0) / 128) & 1) {          // an even number of blocks
            decode_fetch(b1, cv, seg, seg_first, seg_len, t0);
            decode_fetch(b0, cv, seg, seg_first, seg_len, t0 + 128);
            __builtin_amdgcn_sched_barrier(0);
            tile_consume<NJ, ND, true>(t, b1.ka, b1.vt, t0 + 8 * c, 4, scale);
            __builtin_amdgcn_sched_barrier(0);
            t0 += 128;
        } else {
            decode_fetch(b0, cv, seg, seg_first, seg_len, t0);
        }
        while (t0 != last) {                      // the first set holds block t0, an even number of blocks follow
            decode_fetch(b1, cv, seg, seg_first, seg_len, t0 + 128);
            __builtin_amdgcn_sched_barrier(0);
            tile_consume<NJ, ND, true>(t, b0.ka, b0.vt, t0 + 8 * c, 4, scale);
            __builtin_amdgcn_sched_barrier(0);
            decode_fetch(b0, cv, seg, seg_first, seg_len, t0 + 256);
            __builtin_amdgcn_sched_barrier(0);
            tile_consume<NJ, ND, true>(t, b1.ka, b1.vt, t0 + 128 + 8 * c, 4, scale);
            __builtin_amdgcn_sched_barrier(0);
            t0 += 256;
        }
        tile_consume<NJ, ND, true>(t, b0.ka, b0.vt, t0 + 8 * c, 4, scale);
    }

    // merge the four waves: each hands over (m, l, acc) through LDS and combines, in wave order,
    // the dims 16 dt .. of the tiles dt = wave, wave + 4, .., which it then writes
    const int stride = ND * 4 + 2;
    {
        float* dst = lds + ((size_t)wave * 64 + lane) * stride;
        dst[0] = t.m;
        dst[1] = tile_sum(t);
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[2 + dt * 4 + i] = t.acc[dt][i];
    }
    __syncthreads();
    if (!live) return;
    float f[4];
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        f[w] = lds[((size_t)w * 64 + lane) * stride];
        m = w ? fmaxf(m, f[w]) : f[w];
    }
    const float base = (m == -INFINITY) ? 0.f : m;
    float l = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        f[w] = __builtin_amdgcn_exp2f(f[w] - base);
        const float lw = lds[((size_t)w * 64 + lane) * stride + 1] * f[w];
        l = w ? l + lw : lw;
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16_t* o = out + ((size_t)row * heads + head) * head_dim;
    // partial[row][head][split][head_dim + 2]: unnormalised sum, then maximum (in units of log2)
    // and sum of weights
    float* pdst = splits == 1 ? nullptr : partial + (((size_t)row * heads + head) * splits + split) * (head_dim + 2);
#pragma unroll
    for (int dd = 0; dd < (ND + 3) / 4; ++dd) {
        const int dt = dd * 4 + wave;
        if (dt >= ND) break;
        f32x4 a;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float* src = lds + ((size_t)w * 64 + lane) * stride + 2 + dt * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = w ? a[i] + src[i] * f[w] : src[i] * f[w];
        }
        if (splits == 1) {
            uint2 packed;
            packed.x = (uint32_t)f32_to_bf16(a[0] * inv) | ((uint32_t)f32_to_bf16(a[1] * inv) << 16);
            packed.y = (uint32_t)f32_to_bf16(a[2] * inv) | ((uint32_t)f32_to_bf16(a[3] * inv) << 16);
            *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
        } else {
            *reinterpret_cast<f32x4*>(pdst + dt * 16 + 4 * c) = a;
        }
    }
    if (splits > 1 && wave == 0 && c == 0) {
        pdst[head_dim] = m;
        pdst[head_dim + 1] = l;
    }
}

// Decode attention from the raw projections for steps of many rows with short contexts, a wave
// to itself: wave w of a workgroup has row 4 blockIdx.y + w and the kv head of blockIdx.x, norms
// and rotates the row's queries (its 16 columns are the heads of the kv group) and its key,
// writes key and value into the cache, walks all the row's keys in blocks of 32 (the next block
// asked for before this one is multiplied) and writes the output.  No LDS, no barrier, nothing
// merged: where every row has few keys and there are rows enough to fill the chip, four waves
// sharing out one row's prologue and merging their sums spend most of their instructions on
// each other (the kernel above is bound by the issue of its instructions).  The row's block
// table entries are held by the lanes (entry first_entry + lane) and looked up by a shuffle, so
// a row sees at most 64 pages: the caller checks it.  head_dim == 32 NJ, at most 16 heads a kv
// head.  grid (kv_heads * head_tiles, ceil(rows / 4)).
template <int NJ, int ND>
__global__ void __launch_bounds__(256, ND <= 8 ? 2 : 1)      // (two waves a SIMD where the registers allow: a wave on its own waits for every block of its keys)
attention_decode_solo_kernel(bf16_t* __restrict__ out, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                             const int* __restrict__ positions, const int* __restrict__ seq_of_row,
                             const int* __restrict__ tables, int table_width, int page_size, int page_shift,
                             int num_pages, int rows, int heads, int kv_heads, int head_dim, float scale,
                             int window, RawQkv raw) {
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, r = lane % 16, c = lane / 16;
    const int row = blockIdx.y * 4 + wave;
    if (row >= rows) return;                               // (no barrier anywhere: a wave may leave)
    const int group = heads / kv_heads, head_tiles = (group + 15) / 16;
    const int kv_head = blockIdx.x / head_tiles, head_tile = blockIdx.x % head_tiles;
    const int col_head = head_tile * 16 + r;
    const bool live = col_head < group;
    const int head = kv_head * group + (live ? col_head : 0);
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int begin = lo / 32 * 32;
    const int* table = tables + (size_t)seq_of_row[row] * table_width;
    const int first_entry = begin >> page_shift;
    // this lane's table entry, asked for before anything waits
    const int entry_at = min(first_entry + lane, table_width - 1);
    const int my_entry = table[entry_at];
    CacheView cv{k_cache, v_cache, table, table_width, page_size, page_shift, num_pages, kv_heads, head_dim, kv_head};

    const size_t width = (size_t)(heads + 2 * kv_heads) * head_dim;
    const bf16_t* raw_row = raw.qkv ? raw.qkv + (size_t)row * width : nullptr;
    const float* sums_row = raw.partial_sums ? raw.partial_sums + (size_t)row * width : nullptr;
    const float* cos_row = raw.cos ? raw.cos + (size_t)pos * (head_dim / 2) : nullptr;
    const float* sin_row = raw.cos ? raw.sin + (size_t)pos * (head_dim / 2) : nullptr;
    Tile<NJ, ND> t;
    tile_init(t);
    t.pos = live ? pos : -1;
    t.lo = live ? lo : 0;
    const size_t q_off = (size_t)head * head_dim, k_off = (size_t)(heads + kv_head) * head_dim;
    head_from_raw<NJ>(t.q, raw_row ? raw_row + q_off : nullptr, raw.q_norm_w, raw.q_eps, cos_row, sin_row,
                      sums_row ? sums_row + q_off : nullptr, raw.parts, raw.part_stride);
    auto page_of_key = [&](int key) {
        const int page = __shfl(my_entry, (key >> page_shift) - first_entry, 64);
        return (unsigned)page < (unsigned)num_pages ? page : 0;
    };
    if (raw.write_cache) {
        // the row's own key (every lane column computes the same one; column 0 writes it) and value
        Frag kf[NJ];
        head_from_raw<NJ>(kf, raw_row ? raw_row + k_off : nullptr, raw.k_norm_w, raw.k_eps, cos_row, sin_row,
                          sums_row ? sums_row + k_off : nullptr, raw.parts, raw.part_stride);
        const int own_raw = __shfl(my_entry, (pos >> page_shift) - first_entry, 64);
        const bool store = (unsigned)own_raw < (unsigned)num_pages;
        const int slot = pos & (page_size - 1);
        if (store && r == 0) {
            bf16_t* kd = k_cache + (((size_t)own_raw * kv_heads + kv_head) * page_size + slot) * head_dim + c * 8 * NJ;
#pragma unroll
            for (int j = 0; j < NJ; ++j) *reinterpret_cast<uint4*>(kd + j * 8) = kf[j].u;
        }
        if (store) {
            const size_t v_off = (size_t)(heads + kv_heads + kv_head) * head_dim;
            bf16_t* vd = v_cache + ((size_t)own_raw * kv_heads + kv_head) * head_dim * page_size + slot;
            for (int d = lane; d < head_dim; d += 64) {
                bf16_t v;
                if (sums_row) {
                    float a = 0.f;
                    for (int p = 0; p < raw.parts; p += 2) {
                        const bool pair = p + 1 < raw.parts;
                        const float x0 = sums_row[v_off + (size_t)p * raw.part_stride + d];
                        const float x1 = sums_row[v_off + (size_t)(pair ? p + 1 : p) * raw.part_stride + d];
                        a += x0;
                        a += pair ? x1 : 0.f;
                    }
                    v = f32_to_bf16(a);
                } else {
                    v = raw_row[v_off + d];
                }
                vd[(size_t)d * page_size] = cache_value(v);
            }
        }
        // the wave reads its own key and value back with the last block: its stores have to be done
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0)
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }

    // the blocks of 32 keys begin, begin + 32, .. up to the one that holds pos, two sets of
    // registers taking turns (see the kernel above: dealt from the end, nothing asked for twice)
    auto fetch = [&](KeyBlock<NJ, ND>& b, int t0) {
        const int in_page = page_size - 1;
        const int key_k = t0 + 8 * (r / 4) + (r % 4);
        const bf16_t* kp = k_cache + (((size_t)page_of_key(key_k) * kv_heads + kv_head) * page_size + (key_k & in_page)) * head_dim;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                b.ka[u][j].u = *reinterpret_cast<const uint4*>(kp + (size_t)u * 4 * head_dim + c * 8 * NJ + j * 8);
        const int key_v = t0 + 8 * c;
        const bf16_t* vp = v_cache + ((size_t)page_of_key(key_v) * kv_heads + kv_head) * ((size_t)head_dim * page_size) + (key_v & in_page);
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
            b.vt[dt].u = *reinterpret_cast<const uint4*>(vp + (size_t)(dt * 16 + r) * page_size);
    };
    int t0 = begin;
    const int last = pos / 32 * 32;
    {
        KeyBlock<NJ, ND> b0, b1;
        if (((last - t0) / 32) & 1) {                       // an even number of blocks
            fetch(b1, t0);
            fetch(b0, t0 + 32);
            __builtin_amdgcn_sched_barrier(0);
            tile_consume<NJ, ND, true>(t, b1.ka, b1.vt, t0 + 8 * c, 4, scale);
            __builtin_amdgcn_sched_barrier(0);
            t0 += 32;
        } else {
            fetch(b0, t0);
        }
        while (t0 != last) {
            fetch(b1, t0 + 32);
            __builtin_amdgcn_sched_barrier(0);
            tile_consume<NJ, ND, true>(t, b0.ka, b0.vt, t0 + 8 * c, 4, scale);
            __builtin_amdgcn_sched_barrier(0);
            fetch(b0, t0 + 64);
            __builtin_amdgcn_sched_barrier(0);
            tile_consume<NJ, ND, true>(t, b1.ka, b1.vt, t0 + 32 + 8 * c, 4, scale);
            __builtin_amdgcn_sched_barrier(0);
            t0 += 64;
        }
        tile_consume<NJ, ND, true>(t, b0.ka, b0.vt, t0 + 8 * c, 4, scale);
    }
    if (!live) return;
    const float l = tile_sum(t);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16_t* o = out + ((size_t)row * heads + head) * head_dim;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
        uint2 packed;
        packed.x = (uint32_t)f32_to_bf16(t.acc[dt][0] * inv) | ((uint32_t)f32_to_bf16(t.acc[dt][1] * inv) << 16);
        packed.y = (uint32_t)f32_to_bf16(t.acc[dt][2] * inv) | ((uint32_t)f32_to_bf16(t.acc[dt][3] * inv) << 16);
        *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
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
        l += p[head_dim + 1] * __builtin_amdgcn_exp2f(p[head_dim] - base);
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* p = src + (size_t)s * (head_dim + 2);
            a += p[d] * __builtin_amdgcn_exp2f(p[head_dim] - base);
        }
        out[((size_t)row * heads + head) * head_dim + d] = f32_to_bf16(a * inv);
    }
}

// -------------------------------------------------------------------- prefill --
// Which sequence a row block of a step belongs to.  The row blocks of a step are numbered sequence by
// sequence (a sequence of n rows has ceil(n / rows_per_block) of them).  Up to SEQS_WALKED sequences a
// workgroup walks the list by itself (a few scalar loads); beyond, a walk of hundreds of dependent loads
// would take longer than the attention (256 sequences of 8 rows: 499 us a layer), and the workgroup looks
// together: every thread takes a sequence, sums within waves by shuffles and across waves through LDS.
// Both must be called by every thread of the workgroup, before any of them leaves.
#define SEQS_WALKED 16

// All row blocks of the step.
__device__ __forceinline__ int count_row_blocks(const int* __restrict__ row_start, int num_seqs, int rows_per_block) {
    int total = 0;
    if (num_seqs <= SEQS_WALKED) {
        for (int seq = 0; seq < num_seqs; ++seq)
            total += (row_start[seq + 1] - row_start[seq] + rows_per_block - 1) / rows_per_block;
        return total;
    }
    __shared__ int wave_sums[16];
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE, waves = (blockDim.x + TLI_WAVE - 1) / TLI_WAVE;
    for (int s = threadIdx.x; s < num_seqs; s += blockDim.x)
        total += (row_start[s + 1] - row_start[s] + rows_per_block - 1) / rows_per_block;
#pragma unroll
    for (int off = TLI_WAVE / 2; off > 0; off >>= 1) total += __shfl_xor(total, off, TLI_WAVE);
    __syncthreads();                                    // (what an earlier call left there has been read)
    if (lane == 0) wave_sums[wave] = total;
    __syncthreads();
    total = 0;
    for (int w = 0; w < waves; ++w) total += wave_sums[w];
    return total;
}

// Row block `block` of the step: its sequence, that sequence's first row and number of rows, and
// the block's number within the sequence (left in `block`).  False if the step has fewer row blocks.
__device__ __forceinline__ bool find_row_block(int& block, const int* __restrict__ row_start, int num_seqs,
                                               int rows_per_block, int& seq, int& first_row, int& n_rows) {
    if (num_seqs <= SEQS_WALKED) {
        for (seq = 0; seq < num_seqs; ++seq) {
            first_row = row_start[seq];
            n_rows = row_start[seq + 1] - first_row;
            const int blocks = (n_rows + rows_per_block - 1) / rows_per_block;
            if (block < blocks) return true;
            block -= blocks;
        }
        return false;
    }
    __shared__ int wave_totals[16], found[4];
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE, waves = (blockDim.x + TLI_WAVE - 1) / TLI_WAVE;
    __syncthreads();                                    // (what an earlier call left there has been read)
    if (threadIdx.x == 0) found[0] = -1;
    int base = 0;
    for (int s0 = 0; s0 < num_seqs; s0 += blockDim.x) {
        const int s = s0 + threadIdx.x;
        int fr = 0, nr = 0, blocks = 0;
        if (s < num_seqs) {
            fr = row_start[s];
            nr = row_start[s + 1] - fr;
            blocks = (nr + rows_per_block - 1) / rows_per_block;
        }
        int incl = blocks;                              // sum over the lanes up to this one
#pragma unroll
        for (int off = 1; off < TLI_WAVE; off <<= 1) {
            const int up = __shfl_up(incl, off, TLI_WAVE);
            if (lane >= off) incl += up;
        }
        __syncthreads();                                // (the totals of the round before have been read)
        if (lane == TLI_WAVE - 1) wave_totals[wave] = incl;
        __syncthreads();
        int before = base, total = 0;
        for (int w = 0; w < waves; ++w) {
            if (w < wave) before += wave_totals[w];
            total += wave_totals[w];
        }
        before += incl - blocks;                        // row blocks of the sequences before this thread's
        if (blocks > 0 && block >= before && block < before + blocks) {
            found[0] = s;
            found[1] = fr;
            found[2] = nr;
            found[3] = block - before;
        }
        base += total;
        if (block < base) break;                        // (the same for every thread)
    }
    __syncthreads();
    seq = found[0];
    if (seq < 0) return false;
    first_row = found[1];
    n_rows = found[2];
    block = found[3];
    return true;
}

// grid (row blocks upper bound, kv_heads * head_tiles); 256 threads.
// A wave owns CT column tiles; a tile is `rq` consecutive rows of one sequence x
// min(group, 16) heads; the wave's tiles are consecutive in the sequence and share
// every key and value fragment they load.
template <int NJ, int ND, int CT>
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
    const int rows_per_wave = CT * rq, rows_per_block = 4 * rows_per_wave;
    // which sequence and which of its row blocks is this workgroup's?
    int block = blockIdx.x, seq = 0, first_row = 0, n_rows = 0;
    if (!find_row_block(block, row_start, num_seqs, rows_per_block, seq, first_row, n_rows)) return;
    const int local0 = block * rows_per_block + wave * rows_per_wave;   // this wave's first row in the portion
    if (local0 >= n_rows) return;
    const int wave_rows = min(rows_per_wave, n_rows - local0);
    const int start = seq_start[seq];
    // column r of tile ct = (row ct*rq + r / heads_here, head r % heads_here)
    const int col_row = r / heads_here, col_head = head_tile * 16 + r % heads_here;
    const int head = kv_head * group + col_head;

    CacheView cv{k_cache, v_cache, tables + (size_t)seq * table_width, table_width, page_size, page_shift,
                 num_pages, kv_heads, head_dim, kv_head};
    Tile<NJ, ND> t[CT];
    bool live[CT];
    int row[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int local = ct * rq + col_row;
        live[ct] = col_row < rq && local < wave_rows;
        row[ct] = first_row + local0 + (live[ct] ? local : 0);
        const int pos = start + local0 + local;
        tile_init(t[ct]);
        t[ct].pos = live[ct] ? pos : -1;
        t[ct].lo = live[ct] ? (window > 0 ? max(0, pos - window + 1) : 0) : 0;
        tile_load_q(t[ct], q + ((size_t)row[ct] * heads + head) * head_dim, head_dim, live[ct]);
    }

    const int first_pos = start + local0, last_pos = first_pos + wave_rows - 1;
    const int wave_lo = window > 0 ? max(0, first_pos - window + 1) : 0;
    for (int t0 = (wave_lo / 32) * 32; t0 <= last_pos; t0 += 32) tiles_step<NJ, ND, CT>(t, cv, t0, scale);

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (!live[ct]) continue;
        const float l = tile_sum(t[ct]);
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* o = out + ((size_t)row[ct] * heads + head) * head_dim;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            uint2 packed;
            packed.x = (uint32_t)f32_to_bf16(t[ct].acc[dt][0] * inv) | ((uint32_t)f32_to_bf16(t[ct].acc[dt][1] * inv) << 16);
            packed.y = (uint32_t)f32_to_bf16(t[ct].acc[dt][2] * inv) | ((uint32_t)f32_to_bf16(t[ct].acc[dt][3] * inv) << 16);
            *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
        }
    }
}

// ------------------------------------------------- prefill through LDS --
// The same work as attention_prefill_kernel, but the workgroup's four waves share
// every block of KB keys: it is loaded once from the cache into LDS (the next
// block's loads are in flight while the current one is computed) and each wave
// takes its MFMA fragments from there.  Within a 32-key step, row 4c+i of score
// tile u is the key 8c + 4u + i, so the 8 k-slots of lane group c in the output
// MFMA are the 8 consecutive keys 8c..8c+7: one 16-byte read of a value row.
// The head size is ND*16 at compile time.  Needs page_size >= 8.
//
// Keys past the end of a sequence's pages are read from page 0 instead (no
// branches in the loads) and masked: the pools hold finite numbers only (they are
// zero-initialised and written by kernels), so a masked weight of exactly 0 times
// such a value is 0.
template <int NJ, int ND, int CT, int KB>
__device__ __forceinline__ void prefill_lds_block(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ row_start,
    const int* __restrict__ seq_start, int num_seqs, const int* __restrict__ tables, int table_width,
    int page_size, int page_shift, int num_pages, int heads, int kv_heads, float scale_log2, int window,
    int rq, int block, int head_index, const RawQkv& raw) {
    constexpr int HD = ND * 16;
    constexpr int K_PITCH = HD + 8;                   // elements per key row in LDS
    constexpr int V_PITCH = KB + 8;                   // elements per value (dim) row in LDS
    constexpr int K_CHUNKS = KB * HD / 8, V_CHUNKS = HD * KB / 8;      // 16-byte chunks of a block
    constexpr int MAXC = (K_CHUNKS + 255) / 256;
    extern __shared__ uint4 lds_raw[];
    bf16_t* ks = reinterpret_cast<bf16_t*>(lds_raw);  // [KB][K_PITCH]
    bf16_t* vs = ks + KB * K_PITCH;                   // [HD][V_PITCH]
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, r = lane % 16, c = lane / 16;
    const int group = heads / kv_heads;
    const int head_tiles = (group + 15) / 16;
    const int kv_head = head_index / head_tiles, head_tile = head_index % head_tiles;
    const int heads_here = min(16, group - head_tile * 16);
    const int rows_per_wave = CT * rq, rows_per_block = 4 * rows_per_wave;
    int seq = 0, first_row = 0, n_rows = 0;
    if (!find_row_block(block, row_start, num_seqs, rows_per_block, seq, first_row, n_rows))
        return;                                       // the whole workgroup leaves together
    const int start = seq_start[seq];
    const int block0 = block * rows_per_block;        // first row of the workgroup in the portion
    const int block_rows = min(rows_per_block, n_rows - block0);
    const int local0 = block0 + wave * rows_per_wave;
    const int wave_rows = max(0, min(rows_per_wave, n_rows - local0));
    const int col_row = r / heads_here, col_head = head_tile * 16 + r % heads_here;
    const int head = kv_head * group + col_head;
    const int* table = tables + (size_t)seq * table_width;

    Tile<NJ, ND> t[CT];
    bool live[CT];
    int row[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int local = ct * rq + col_row;
        live[ct] = col_row < rq && local < wave_rows;
        row[ct] = first_row + (live[ct] ? local0 + local : 0);
        const int pos = start + local0 + local;
        tile_init(t[ct]);
        t[ct].pos = live[ct] ? pos : -1;
        t[ct].lo = live[ct] ? (window > 0 ? max(0, pos - window + 1) : 0) : 0;
        if (NJ * 2 == ND && raw.qkv) {
            // the query from the raw projections: this row's head, normed and rotated here
            // (an idle column computes on the first row of the portion; it is masked)
            const int at = live[ct] ? pos : start;
            const float* cos_row = raw.cos ? raw.cos + (size_t)at * (HD / 2) : nullptr;
            const float* sin_row = raw.cos ? raw.sin + (size_t)at * (HD / 2) : nullptr;
            head_from_raw<NJ>(t[ct].q, raw.qkv + ((size_t)row[ct] * (heads + 2 * kv_heads) + head) * HD,
                              raw.q_norm_w, raw.q_eps, cos_row, sin_row);
        } else {
            tile_load_q(t[ct], q + ((size_t)row[ct] * heads + head) * HD, HD, live[ct]);
        }
    }
    // keys the workgroup walks, and those this wave needs
    const int wg_first = start + block0, wg_last = wg_first + block_rows - 1;
    const int wg_lo = window > 0 ? max(0, wg_first - window + 1) : 0;
    const int wave_first = start + local0, wave_last = wave_first + wave_rows - 1;
    const int wave_lo = window > 0 ? max(0, wave_first - window + 1) : 0;
    // every key in [full_lo, full_hi] is seen by every live column of this wave
    const int full_lo = window > 0 ? max(0, wave_last - window + 1) : 0, full_hi = wave_first;

    // staging plan of this thread: chunk e is key row (tid + 256 e) / (HD/8) of the block
    // for keys, and dim row (tid + 256 e) / (KB/8) for values; fixed over the blocks.
    // (A thread without a chunk e asks for chunk 0 once more and does not store it: no
    // load below is under a branch, or the compiler would wait for all loads in flight at
    // the next use and the prefetching would be undone.)
    int k_key[MAXC], k_dch[MAXC], k_lds[MAXC], v_lds[MAXC];
    bool mine[MAXC];
    size_t v_dim_off[MAXC];
    const int v_g8 = tid % (KB / 8);                  // this thread's group of 8 keys in every value row
    const size_t head_k = (size_t)kv_head * page_size * HD, page_k = (size_t)kv_heads * page_size * HD;
    const size_t head_v = (size_t)kv_head * HD * page_size, page_v = (size_t)kv_heads * HD * page_size;
#pragma unroll
    for (int e = 0; e < MAXC; ++e) {
        mine[e] = K_CHUNKS % 256 == 0 || tid + e * 256 < K_CHUNKS;
        const int idx = mine[e] ? tid + e * 256 : 0;
        k_key[e] = idx / (HD / 8);
        k_dch[e] = (idx % (HD / 8)) * 8;
        k_lds[e] = k_key[e] * K_PITCH + k_dch[e];
        const int d = idx / (KB / 8);
        v_lds[e] = d * V_PITCH + v_g8 * 8;
        v_dim_off[e] = (size_t)d * page_size;
    }
    u32x4 kreg[MAXC], vreg[MAXC];
    // The pages of a block are looked up one block before its keys and values are asked
    // for, so that an address never waits for a table entry.  A key without a page (past
    // the table, or released) reads page 0: it lies outside what any row sees.
    int k_page[MAXC], v_page;
    auto page_of = [&](int key) {
        const int page = table[min(key >> page_shift, table_width - 1)];
        return (unsigned)page < (unsigned)num_pages ? page : 0;
    };
    auto lookup = [&](int t0) {
#pragma unroll
        for (int e = 0; e < MAXC; ++e) k_page[e] = page_of(t0 + k_key[e]);
        v_page = page_of(t0 + v_g8 * 8);
    };
    auto fetch = [&](int t0) {
        const int vkey = t0 + v_g8 * 8;
        const bf16_t* vbase = v_cache + (size_t)v_page * page_v + head_v + (vkey & (page_size - 1));
#pragma unroll
        for (int e = 0; e < MAXC; ++e) {
            const int key = t0 + k_key[e];
            kreg[e] = *reinterpret_cast<const u32x4*>(
                k_cache + (size_t)k_page[e] * page_k + head_k + (size_t)(key & (page_size - 1)) * HD + k_dch[e]);
            vreg[e] = *reinterpret_cast<const u32x4*>(vbase + v_dim_off[e]);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int e = 0; e < MAXC; ++e) {
            if (mine[e]) {
                *reinterpret_cast<u32x4*>(ks + k_lds[e]) = kreg[e];
                *reinterpret_cast<u32x4*>(vs + v_lds[e]) = vreg[e];
            }
        }
    };
    static_assert(K_CHUNKS == V_CHUNKS, "keys and values of a block have as many chunks");

    // LDS offsets of this lane's fragments inside a 32-key step
    int ka_off[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) ka_off[u] = (8 * (r / 4) + 4 * u + (r % 4)) * K_PITCH + c * 8 * NJ;
    const int vt_off = r * V_PITCH + 8 * c;

    int t0 = (wg_lo / KB) * KB;
    const int t_last = (wg_last / KB) * KB;             // the last block; asked for again rather than branching
    lookup(t0);
    fetch(t0);
    lookup(min(t0 + KB, t_last));
    for (; t0 <= wg_last; t0 += KB) {
        __syncthreads();                 // everyone has finished reading the previous block
        stage();
        __syncthreads();
        fetch(min(t0 + KB, t_last));
        lookup(min(t0 + 2 * KB, t_last));
#pragma unroll
        for (int sub = 0; sub < KB / 32; ++sub) {
            const int s0 = t0 + sub * 32;
            if (wave_rows <= 0 || s0 > wave_last || s0 + 31 < wave_lo) continue;   // nothing this wave sees
            Frag ka[2][NJ], vt[ND];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    if (c * 8 * NJ + j * 8 < HD)
                        ka[u][j].u = *reinterpret_cast<const uint4*>(ks + sub * 32 * K_PITCH + ka_off[u] + j * 8);
                    else
                        ka[u][j].u = make_uint4(0, 0, 0, 0);
                }
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
                vt[dt].u = *reinterpret_cast<const uint4*>(vs + dt * 16 * V_PITCH + vt_off + sub * 32);
            if (s0 >= full_lo && s0 + 31 <= full_hi)
                tiles_consume<NJ, ND, CT, false>(t, ka, vt, s0 + 8 * c, 4, scale_log2);
            else
                tiles_consume<NJ, ND, CT, true>(t, ka, vt, s0 + 8 * c, 4, scale_log2);
        }
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (!live[ct]) continue;
        const float l = tile_sum(t[ct]);
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* o = out + ((size_t)row[ct] * heads + head) * HD;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            uint2 packed;
            packed.x = pack_bf16x2(t[ct].acc[dt][0] * inv, t[ct].acc[dt][1] * inv);
            packed.y = pack_bf16x2(t[ct].acc[dt][2] * inv, t[ct].acc[dt][3] * inv);
            *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
        }
    }
}

typedef __attribute__((address_space(3))) void lds_void_t;

// -------------------------- prefill, copied straight into LDS, phases overlapped --
// The same work for heads of 64 and 128 (ND = 4, 8; NJ = ND/2), with the keys and values
// copied from the cache into LDS by the memory pipeline itself (global_load_lds_dwordx4: lane
// l of a wave writes the 16 bytes it asked for at LDS base + 16 l, no register holds them
// meanwhile), 32 keys a step through four buffers.  Such a copy leaves no room for padding
// between rows, so rows are swizzled instead: a lane chooses which 16 bytes of the cache it
// asks for, and asks for those that belong at its place.  Keys: row = key, 16-byte chunk q of
// the row lies at chunk q ^ f(key) with f(key) = (key & 3) | ((key >> 3) & 3) << 2 (halved for
// rows of 8 chunks): the 16 lanes that read one chunk column for an MFMA operand (keys
// 8 (r/4) + 4 u + r%4) then hit 16 different bank groups.  Values: four planes of 8 keys, a
// plane [dim][8 keys]: the 16 lanes that read one plane for an MFMA operand take 256 bytes in
// a row.
// The phases of a wave's step are overlapped: while the matrix pipeline works on the
// scores of step i+1 the vector units turn the exponents of step i into weights, and while it
// adds up the values of step i they turn the scores of step i+1 into exponents.  A wave
// issues one instruction at a time, and an MFMA that waits for the pipeline holds up what
// follows it, so the two kinds stand interleaved in the program.
//   top of iteration i:  block i+1 has landed (the copies of block i+2 may still be under way),
//                        barrier, start the copy of block i+3 into the buffer that block i-1 left
//   then:                key fragments of step i+1 and value fragments of step i from LDS,
//                        weights of step i, scores of step i+1, output of step i, exponents of
//                        step i+1 (its bases may move: the sums are rescaled after the output)
// A wave sees the steps a..b of the workgroup's 0..n-1 (late rows see more keys than early
// ones); before and after them it only takes part in the barriers and the copies.
// KG = 2: the workgroup has two sets of four waves with the same rows; a block brings 64 keys,
// of which the first set takes the first 32 and the second set the rest, and the second set's
// sums are added to the first's through LDS at the end.  A workgroup then walks its keys in
// half as many rounds, which is what counts where the longest workgroups decide the time (a
// prompt of 2,048 tokens: the last rows walk 64 steps of 32 keys while the chip has room for
// every workgroup at once).
// (Workgroups of eight waves with twice the rows, which ask the L2 caches for every key half as
// often, were measured 3 to 6% slower than two workgroups of four.)
template <int NJ, int ND, int CT, int KG>
__device__ __forceinline__ void prefill_pipe_block(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ row_start,
    const int* __restrict__ seq_start, int num_seqs, const int* __restrict__ tables, int table_width,
    int page_size, int page_shift, int num_pages, int heads, int kv_heads, float scale_log2, int window,
    int rq, int block, int head_index, const RawQkv& raw) {
    static_assert(ND == 2 * NJ && (ND == 4 || ND == 8), "heads of 64 or 128");
    constexpr int KB = 32;                            // keys of a step
    constexpr int BK = KB * KG;                       // keys of a block: a step for each set of waves
    constexpr int WAVES = 4 * KG;
    constexpr int HD = ND * 16;
    constexpr int CR = HD / 8;                        // 16-byte chunks of a key row
    constexpr int KI = BK * CR / (64 * WAVES), VI = HD * (BK / 8) / (64 * WAVES);     // copies a wave issues for a block: keys, values
    static_assert(KI >= 1 && VI >= 1, "every wave takes part in the copies");
    constexpr int PER = KI + VI;
    constexpr int TILE = BK * HD;                     // elements of a block's keys (and of its values)
    extern __shared__ uint4 lds_raw[];
    bf16_t* lds = reinterpret_cast<bf16_t*>(lds_raw); // buffer b: keys at b * 2 TILE, values TILE further
    const int tid = threadIdx.x, lane = tid % 64, wave = (tid / 64) % 4, r = lane % 16, c = lane / 16;
    const int group = heads / kv_heads;
    const int head_tiles = (group + 15) / 16;
    const int kv_head = head_index / head_tiles, head_tile = head_index % head_tiles;
    const int heads_here = min(16, group - head_tile * 16);
    const int rows_per_wave = CT * rq, rows_per_block = 4 * rows_per_wave;
    int seq = 0, first_row = 0, n_rows = 0;
    if (!find_row_block(block, row_start, num_seqs, rows_per_block, seq, first_row, n_rows))
        return;                                       // the whole workgroup leaves together
    const int start = seq_start[seq];
    const int block0 = block * rows_per_block;        // first row of the workgroup in the portion
    const int block_rows = min(rows_per_block, n_rows - block0);
    const int local0 = block0 + wave * rows_per_wave;
    const int wave_rows = max(0, min(rows_per_wave, n_rows - local0));
    const int col_row = r / heads_here, col_head = head_tile * 16 + r % heads_here;
    const int head = kv_head * group + col_head;
    const int* table = tables + (size_t)seq * table_width;

    Tile<NJ, ND> t[CT];
    bool live[CT];
    int row[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int local = ct * rq + col_row;
        live[ct] = col_row < rq && local < wave_rows;
        row[ct] = first_row + (live[ct] ? local0 + local : 0);
        const int pos = start + local0 + local;
        tile_init(t[ct]);
        t[ct].pos = live[ct] ? pos : -1;
        t[ct].lo = live[ct] ? (window > 0 ? max(0, pos - window + 1) : 0) : 0;
        if (raw.qkv) {
            const int at = live[ct] ? pos : start;
            const float* cos_row = raw.cos ? raw.cos + (size_t)at * (HD / 2) : nullptr;
            const float* sin_row = raw.cos ? raw.sin + (size_t)at * (HD / 2) : nullptr;
            head_from_raw<NJ>(t[ct].q, raw.qkv + ((size_t)row[ct] * (heads + 2 * kv_heads) + head) * HD,
                              raw.q_norm_w, raw.q_eps, cos_row, sin_row);
        } else {
            tile_load_q(t[ct], q + ((size_t)row[ct] * heads + head) * HD, HD, live[ct]);
        }
    }
    const int wg_first = start + block0, wg_last = wg_first + block_rows - 1;
    const int wg_lo = window > 0 ? max(0, wg_first - window + 1) : 0;
    const int wave_first = start + local0, wave_last = wave_first + wave_rows - 1;
    const int wave_lo = window > 0 ? max(0, wave_first - window + 1) : 0;
    // The blocks: the workgroup's 0..n-1 from key T0.  Block i holds step KG i + set for each set of
    // waves; this wave's steps are those of its blocks a..b, of which the steps f0..f1-1 are seen
    // whole by every row of the wave (the others need the comparison of every key with the row's range).
    const int wave_u = __builtin_amdgcn_readfirstlane(tid / 64);     // the wave, in a scalar register (for the copies' addresses)
    const int set = wave_u / 4;                       // which of the KG sets of four waves
    const int T0 = (wg_lo / BK) * BK;
    const int n = (wg_last - T0) / BK + 1;
    const int full_lo = window > 0 ? max(0, wave_last - window + 1) : 0, full_hi = wave_first;
    const int step_lo = (wave_lo - T0) / KB, step_hi = (wave_last - T0) / KB;      // the wave's steps of 32 keys
    const bool any = wave_rows > 0 && step_hi >= set && (step_lo - set + KG - 1) / KG <= (step_hi - set) / KG;
    // (the same for a whole wave, and said so: the loops below then run on scalar registers)
    const int a = __builtin_amdgcn_readfirstlane(any ? max(0, step_lo - set + KG - 1) / KG : n + 1);
    const int b = __builtin_amdgcn_readfirstlane(any ? (step_hi - set) / KG : n);
    const int f0 = __builtin_amdgcn_readfirstlane(full_lo <= T0 ? 0 : (full_lo - T0 + KB - 1) / KB);
    const int f1 = __builtin_amdgcn_readfirstlane((full_hi - T0 + 1) / KB);
    auto whole = [&](int block) { return KG * block + set >= f0 && KG * block + set < f1; };
    auto first_key = [&](int block) { return T0 + (KG * block + set) * KB; };      // of this wave's step in a block

    // Copy w = WAVES e + wave of a block moves 64 x 16 bytes: for keys the KPC rows from w KPC of the
    // block (lane l: row l / CR, the chunk that belongs at chunk l % CR of that row); for values
    // 64 dims of the plane w / WPP (lane l: dim
    // (w % WPP) 64 + l, the plane's 8 keys).  A page holds at least 8 keys, so what copy e moves of
    // the keys and of the values lies in one page.  An address is a base in scalar registers plus
    // an offset that a lane keeps for the whole kernel.
    constexpr int KPC = 64 / CR;                      // key rows a copy moves (4 or 8)
    constexpr int WPP = HD / 64;                      // copies that make up a plane of values
    static_assert(KI == VI && KPC * WPP == 8, "copy e of the keys and of the values share a page");
    auto swz_key = [](int key) {
        const int f = (key & 3) | (((key >> 3) & 3) << 2);
        return CR == 16 ? f : f >> 1;
    };
    uint32_t k_loff[KI], v_loff[VI];
#pragma unroll
    for (int e = 0; e < KI; ++e) {
        const int w = e * WAVES + wave_u, first = w * KPC;  // the copy's first key in the block
        const int k_row = first + lane / CR;
        k_loff[e] = (uint32_t)((((first & (page_size - 1)) + lane / CR) * HD + ((lane % CR) ^ swz_key(k_row)) * 8) *
                               sizeof(bf16_t));
        v_loff[e] = (uint32_t)(((size_t)((w % WPP) * 64 + lane) * page_size + ((first & ~7) & (page_size - 1))) *
                               sizeof(bf16_t));
    }
    const uint64_t page_bytes = (uint64_t)kv_heads * page_size * HD * sizeof(bf16_t);     // of the keys, and of the values
    const uint64_t head_bytes = (uint64_t)kv_head * page_size * HD * sizeof(bf16_t);
    // 64 entries of the block table at a time live in the lanes of one register (entry
    // tab_first + l in lane l, those that name no page made 0: such keys are masked); a copy takes
    // its page from there with v_readlane.  The register is filled again every 512 keys, which
    // walk at most 64 entries (pages of 8 keys).
    int tab_first = 0, tab_pages = 0;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t*)lds;
    // one copy of 64 x 16 bytes: LDS place (bytes from the start of the buffers) <- base + the lane's offset
    auto dma = [&](uint32_t lds_byte, uint32_t lane_off, uint64_t base) {
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     ::"s"(lds_base), "s"(lds_byte), "v"(lane_off), "s"(base)
                     : "m0", "scc", "memory");
    };
    // start the copies of block `step` < n into its buffer (called for every block in turn)
    auto copy = [&](int step) {
        const int t0 = T0 + step * BK;
        if ((step & (16 / KG - 1)) == 0) {
            tab_first = t0 >> page_shift;
            // (loaded and waited for in assembly, like the copies: the compiler then knows of no load
            // in the loop and leaves the counting of those in flight to the waits written here)
            int page;
            asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)"
                         : "=v"(page)
                         : "v"(table + min(tab_first + lane, table_width - 1))
                         : "memory");
            tab_pages = (unsigned)page < (unsigned)num_pages ? page : 0;
        }
        const uint32_t kb = (uint32_t)(step & 3) * (uint32_t)(2 * TILE * sizeof(bf16_t));
        const uint64_t in_page = (uint64_t)(t0 & (page_size - 1) & ~(BK - 1));     // pages of more keys than a block
        const uint64_t k_base = (uint64_t)(uintptr_t)k_cache + head_bytes + in_page * (HD * sizeof(bf16_t));
        const uint64_t v_base = (uint64_t)(uintptr_t)v_cache + head_bytes + in_page * sizeof(bf16_t);
#pragma unroll
        for (int e = 0; e < KI; ++e) {
            const int entry = (t0 + (e * WAVES + wave_u) * KPC) >> page_shift;
            const uint64_t page_off = (uint64_t)(uint32_t)__builtin_amdgcn_readlane(tab_pages, entry - tab_first) * page_bytes;
            dma(kb + (e * WAVES + wave_u) * 1024, k_loff[e], k_base + page_off);
            dma(kb + (uint32_t)(TILE * sizeof(bf16_t)) + (e * WAVES + wave_u) * 1024, v_loff[e], v_base + page_off);
        }
    };
    // the top of iteration i.  In flight are this wave's copies of block i+1 and, if there is one,
    // of block i+2, in that order: past the last block nothing is copied (copying the last one again
    // instead was a third more copies for a workgroup of average length at 2,048 tokens), and the
    // wait counts what is there.  (i and the number of blocks are in scalar registers: the
    // branches are the same for the whole workgroup.)
    const int n_s = __builtin_amdgcn_readfirstlane(n);
    auto top = [&](int i) {
        if (i + 2 < n_s)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER) : "memory");     // this wave's part of block i+1 has landed
        else
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                               // everyone's has, and nobody reads block i-1 any more
        if (i + 3 < n_s) copy(i + 3);
    };

    // LDS offsets (elements) of this lane's fragments in a buffer: the keys from row 32 set of the
    // block (values: plane 4 set + c, dim 16 dt + r)
    int ka_row[2], ka_col[NJ];
#pragma unroll
    for (int u = 0; u < 2; ++u) ka_row[u] = (KB * set + 8 * (r / 4) + 4 * u + (r % 4)) * HD;
#pragma unroll
    for (int j = 0; j < NJ; ++j) ka_col[j] = ((c * NJ + j) ^ (CR == 16 ? r : r >> 1)) * 8;
    const int vt_at = TILE + ((4 * set + c) * HD + r) * 8;
    auto keys_of = [&](int step, Frag (&ka)[2][NJ]) {
        const bf16_t* ks = lds + (size_t)(step & 3) * 2 * TILE;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int j = 0; j < NJ; ++j) ka[u][j].u = *reinterpret_cast<const uint4*>(ks + ka_row[u] + ka_col[j]);
    };
    auto values_of = [&](int step, Frag (&vt)[ND]) {
        const bf16_t* vs = lds + (size_t)(step & 3) * 2 * TILE + vt_at;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) vt[dt].u = *reinterpret_cast<const uint4*>(vs + dt * 16 * 8);
    };

    f32x4 ex[CT][2];                                  // the exponents of the step whose weights come next
    copy(0);
    if (1 < n_s) copy(1);
    int i = -1;
    for (; i < a - 1; ++i) top(i);                    // blocks before this wave's keys
    if (a <= b) {
        {                                             // i == a - 1: the scores of the wave's first step
            top(i);
            Frag ka[2][NJ];
            keys_of(a, ka);
            tiles_scores<NJ, ND, CT>(t, ka, ex);
            if (whole(a))
                tiles_exponents<NJ, ND, CT, false>(t, ex, first_key(a) + 8 * c, 4, scale_log2);
            else
                tiles_exponents<NJ, ND, CT, true>(t, ex, first_key(a) + 8 * c, 4, scale_log2);
            ++i;
        }
        auto round = [&](auto MASK_T) {
            constexpr bool MASK = decltype(MASK_T)::value;
            top(i);
            Frag ka[2][NJ], vt[ND], pb[CT];
            f32x4 sc[CT][2];
            keys_of(i + 1, ka);
            values_of(i, vt);
            tiles_pack<CT>(ex, pb);
            tiles_scores<NJ, ND, CT>(t, ka, sc);
            tiles_output<NJ, ND, CT>(t, vt, pb);
            tiles_exponents<NJ, ND, CT, MASK>(t, sc, first_key(i + 1) + 8 * c, 4, scale_log2);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int u = 0; u < 2; ++u) ex[ct][u] = sc[ct][u];
        };
        while (i < b) {
            for (; i < b && whole(i + 1); ++i) round(std::false_type{});     // the step after i is seen whole
            for (; i < b && !whole(i + 1); ++i) round(std::true_type{});
        }
        {                                             // i == b: the output of the wave's last step
            top(i);
            Frag vt[ND], pb[CT];
            values_of(b, vt);
            tiles_pack<CT>(ex, pb);
            tiles_output<NJ, ND, CT>(t, vt, pb);
            ++i;
        }
    }
    for (; i < n; ++i) top(i);                        // blocks after this wave's keys
    // the copies that the last rounds started land before anything else uses the buffers
    __builtin_amdgcn_s_waitcnt(0x0F70);

    if constexpr (KG > 1) {
        // the other sets hand their sums over through LDS ([set - 1][wave][tile][lane]: base, sum of
        // the weights, sums of the values), the first set adds them up in set order
        constexpr int STRIDE = ND * 4 + 2;
        static_assert((size_t)(KG - 1) * 4 * CT * 64 * STRIDE * sizeof(float) <= (size_t)4 * 2 * TILE * sizeof(bf16_t),
                      "the sums fit the buffers");
        float* sums = reinterpret_cast<float*>(lds_raw);
        __syncthreads();                                  // nobody reads keys or values any more
        if (set > 0) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                float* dst = sums + ((((size_t)(set - 1) * 4 + wave) * CT + ct) * 64 + lane) * STRIDE;
                dst[0] = t[ct].m;
                dst[1] = tile_sum(t[ct]);
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) dst[2 + dt * 4 + i4] = t[ct].acc[dt][i4];
            }
        }
        __syncthreads();
        if (set > 0) return;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float m = t[ct].m;
            for (int other = 1; other < KG; ++other)
                m = fmaxf(m, sums[((((size_t)(other - 1) * 4 + wave) * CT + ct) * 64 + lane) * STRIDE]);
            const float base = (m == -INFINITY) ? 0.f : m;
            float f = __builtin_amdgcn_exp2f(t[ct].m - base);
            float l = tile_sum(t[ct]) * f;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) t[ct].acc[dt][i4] *= f;
            for (int other = 1; other < KG; ++other) {
                const float* src = sums + ((((size_t)(other - 1) * 4 + wave) * CT + ct) * 64 + lane) * STRIDE;
                f = __builtin_amdgcn_exp2f(src[0] - base);
                l += src[1] * f;
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) t[ct].acc[dt][i4] += src[2 + dt * 4 + i4] * f;
            }
            t[ct].ls = (f32x4){l, l, l, l};
            t[ct].l = 0.f;
        }
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (!live[ct]) continue;
        const float l = tile_sum(t[ct]);
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* o = out + ((size_t)row[ct] * heads + head) * HD;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            uint2 packed;
            packed.x = pack_bf16x2(t[ct].acc[dt][0] * inv, t[ct].acc[dt][1] * inv);
            packed.y = pack_bf16x2(t[ct].acc[dt][2] * inv, t[ct].acc[dt][3] * inv);
            *reinterpret_cast<uint2*>(o + dt * 16 + 4 * c) = packed;
        }
    }
}

// With raw.qkv the queries are taken from the raw projections (normed and rotated here, q
// is not read); needs head_dim == 32*NJ.  DMA: keys and values are copied straight into LDS
// (prefill_pipe_block; heads of 64 and 128, KB = 32).
// grid (row blocks, kv_heads * head_tiles).  Row blocks late in a sequence walk more keys
// than early ones; `pair` says how the work is evened out: 1: (ceil(row blocks / 2), ...)
// workgroups that each take block (last - b) and then block b; 2: long blocks placed beside
// short ones on a compute unit; 3: long blocks first; 0: as the grid says.
template <int NJ, int ND, int CT, int KB, bool DMA, int KG = 1>
__global__ void __launch_bounds__(KG * 256, (KG == 1 && ND <= 8 && (CT == 2 || DMA)) ? 2 : 1)
attention_prefill_lds_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                             const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                             const int* __restrict__ row_start, const int* __restrict__ seq_start,
                             int num_seqs, const int* __restrict__ tables, int table_width, int page_size,
                             int page_shift, int num_pages, int heads, int kv_heads,
                             float scale_log2, int window, int rq, int pair, RawQkv raw) {
    const int rows_per_block = 4 * CT * rq;
    const int total = count_row_blocks(row_start, num_seqs, rows_per_block);
    const int head_count = gridDim.y;
    // the row block and head (and for pair = 1 a second row block) of this workgroup
    int rb, hd_i = blockIdx.y, rb2 = -1;
    if (pair == 2) {
        // All workgroups are resident at once, two a compute unit, and late row blocks walk
        // more keys than early ones.  Workgroups are handed to the compute units in order
        // of their linear index, so index L and index L + total/2 tend to share a unit: the
        // second half of the indices gets the row blocks in reverse order (and the other
        // half of the heads), which puts a long block beside a short one.
        const int half = total * head_count / 2;
        if (blockIdx.x >= total) return;                       // the grid's slack
        const int lin = blockIdx.y * total + blockIdx.x;       // index among the real workgroups
        if (head_count % 2 == 0) {
            const int round = lin / half, p = lin % half;
            rb = round == 0 ? p % total : total - 1 - p % total;
            hd_i = p / total + round * (head_count / 2);
        } else {
            rb = blockIdx.x;
        }
    } else if (pair == 3) {
        // Long row blocks first: workgroups are handed out in the order of their index as
        // compute units become free, so the short blocks fill the gaps the long ones leave.
        // The heads vary fastest, so that what runs at the same time walks similar key ranges.
        if (blockIdx.x >= total) return;                      // the grid's slack
        const int idx = blockIdx.y * total + blockIdx.x;      // index among the real workgroups
        rb = total - 1 - idx / head_count;
        hd_i = idx % head_count;
    } else {
        const int first = blockIdx.x, second = pair ? total - 1 - first : first;
        if (first >= total || first > second) return;
        rb = second;
        if (second != first) rb2 = first;
    }
    const int passes = rb2 < 0 ? 1 : 2;
    for (int pass = 0; pass < passes; ++pass) {
        if (pass) __syncthreads();                            // (the buffers are used again)
        const int block = pass ? rb2 : rb;
        if constexpr (DMA)
            prefill_pipe_block<NJ, ND, CT, KG>(q, out, k_cache, v_cache, row_start, seq_start, num_seqs, tables,
                                                  table_width, page_size, page_shift, num_pages, heads, kv_heads,
                                                  scale_log2, window, rq, block, hd_i, raw);
        else
            prefill_lds_block<NJ, ND, CT, KB>(q, out, k_cache, v_cache, row_start, seq_start, num_seqs, tables,
                                              table_width, page_size, page_shift, num_pages, heads, kv_heads,
                                              scale_log2, window, rq, block, hd_i, raw);
    }
}

// ------------------------------------------------------------------------ host --
static const float LOG2E = 1.4426950408889634f;     // scores are kept in units of log2

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
static int launch_decode(const void* q, void* out, float* partial, void* k_cache, void* v_cache,
                         const int* positions, const int* seq_of_row, const int* tables, int table_width,
                         int page_size, int num_pages, int rows, int heads, int kv_heads, int head_dim,
                         float scale, int window, int splits, int keys_per_split, const RawQkv* raw,
                         void* stream) {
    if (rows <= 0) return 0;
    if (check_common("attention_decode", heads, kv_heads, head_dim, page_size, table_width, num_pages)) return 1;
    if (splits == 0) {
        // a wave a row: from the raw projections only, heads of 64, 128 or 256, the keys that a row
        // sees within 64 pages
        const int group0 = heads / kv_heads, tiles0 = (group0 + 15) / 16;
        if (!raw || head_dim % 64 || head_dim == 192 || group0 > 16 || page_size < 8)
            return tli_fail("attention_decode, a wave a row: from raw projections with heads of 64, 128 or 256, at "
                            "most 16 heads a kv head, pages of at least 8");
        // (a wave keeps 64 table entries; a window that begins inside a page and the rounding to blocks
        // of 32 keys take up to two more than the keys themselves)
        if (keys_per_split <= 0 || keys_per_split > 60 * page_size)
            return tli_fail("attention_decode, a wave a row: %d keys in pages of %d are more than the 60 pages a wave "
                            "keeps the table entries of", keys_per_split, page_size);
        if ((rows + 3) / 4 > 65535) return tli_fail("attention_decode: %d rows exceed the grid limit", rows);
        dim3 grid0(kv_heads * tiles0, (rows + 3) / 4);
        hipStream_t s0 = (hipStream_t)stream;
        const int shift0 = log2_exact(page_size);
#define SOLO(NJ, ND)                                                                                              \
    attention_decode_solo_kernel<NJ, ND><<<grid0, 256, 0, s0>>>((bf16_t*)out, (bf16_t*)k_cache, (bf16_t*)v_cache,   \
        positions, seq_of_row, tables, table_width, page_size, shift0, num_pages, rows, heads, kv_heads, head_dim, \
        scale * LOG2E, window, *raw)
        if (head_dim == 64) SOLO(2, 4);
        else if (head_dim == 128) SOLO(4, 8);
        else SOLO(8, 16);
#undef SOLO
        return tli_check_launch("attention_decode_solo");
    }
    if (splits < 1 || splits > 65535 || keys_per_split <= 0 || keys_per_split % 128)
        return tli_fail("attention_decode: %d splits of %d keys (keys per split must be a multiple of 128)",
                        splits, keys_per_split);
    if (splits > 1 && !partial) return tli_fail("attention_decode: splits need a partial buffer");
    if (rows > 65535) return tli_fail("attention_decode: %d rows exceed the grid limit", rows);
    if (page_size < 8) return tli_fail("attention_decode: pages of %d keys, the kernel takes pages of at least 8", page_size);
    hipStream_t s = (hipStream_t)stream;
    const int group = heads / kv_heads, head_tiles = (group + 15) / 16;
    if (raw && (head_dim % 64 || group > 16))
        return tli_fail("attention_decode from raw projections: head_dim %d must be a multiple of 64 and "
                        "heads per kv head (%d) at most 16", head_dim, group);
    dim3 grid(kv_heads * head_tiles, rows, splits);
    const int shift = log2_exact(page_size);
    // the table entries of one split are kept in LDS
    const size_t seg_bytes = ((((size_t)(keys_per_split >> shift) + 2) + 3) & ~(size_t)3) * sizeof(int);      // (16-byte aligned: the prologue's exchange comes behind it)
    if (seg_bytes > 8192)
        return tli_fail("attention_decode: %d keys per split in pages of %d are more than 2046 pages; use more splits",
                        keys_per_split, page_size);
    const RawQkv none{};
#define ARGS (const bf16_t*)q, (bf16_t*)out, partial, (bf16_t*)k_cache, (bf16_t*)v_cache, positions, seq_of_row, \
             tables, table_width, page_size, shift, num_pages, heads, kv_heads, head_dim, scale * LOG2E, window, \
             splits, keys_per_split
#define LDS_BYTES(ND) (4 * 64 * (ND * 4 + 2) * sizeof(float) + seg_bytes + (raw ? 2 * 4 * 16 * sizeof(float) + (ND / 2) * 64 * sizeof(uint4) : 0))
    // (more than 64 KiB of LDS, which the widest heads need, has to be allowed for a kernel once)
#define ONE(NJ, ND, F, R)                                                                                   \
    {                                                                                                       \
        auto kernel = attention_decode_kernel<NJ, ND, F>;                                                   \
        const size_t bytes = LDS_BYTES(ND);                                                                 \
        static bool allowed = false;                                                                        \
        if (bytes > 65536 && !allowed) {                                                                    \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,        \
                                    (int)bytes + 8192) != hipSuccess)                                       \
                return tli_fail("attention_decode: cannot have %zu bytes of LDS", bytes);                   \
            allowed = true;                                                                                 \
        }                                                                                                   \
        kernel<<<grid, 256, bytes, s>>>(ARGS, R);                                                           \
    }
#define CALL(NJ, ND)                                                                                        \
    if (raw) ONE(NJ, ND, NJ * 2 == ND, *raw)                                                                \
    else ONE(NJ, ND, false, none)
    DISPATCH_HEAD_DIM(CALL)
#undef ONE
#undef CALL
#undef LDS_BYTES
#undef ARGS
    if (tli_check_launch("attention_decode")) return 1;
    if (splits > 1) {
        attention_merge_splits_kernel<<<dim3(heads, rows), 64, 0, s>>>(partial, (bf16_t*)out, heads, head_dim, splits);
        return tli_check_launch("attention_merge_splits");
    }
    return 0;
}

extern "C" int tli_attention_decode_bf16(
    const void* q, void* out, float* partial, const void* k_cache, const void* v_cache,
    const int* positions, const int* seq_of_row, const int* tables, int table_width, int page_size,
    int num_pages, int rows, int heads, int kv_heads, int head_dim, float scale, int window,
    int splits, int keys_per_split, void* stream) {
    return launch_decode(q, out, partial, (void*)k_cache, (void*)v_cache, positions, seq_of_row, tables,
                         table_width, page_size, num_pages, rows, heads, kv_heads, head_dim, scale, window,
                         splits, keys_per_split, nullptr, stream);
}

// Decode attention straight from the raw projections qkv [rows][(heads + 2 kv_heads) * head_dim]:
// per-head norm (weights may be null), rotation (cos/sin [table_positions][head_dim/2] or null:
// the whole head is rotated), the row's key and value into the cache (write_cache), then
// attention as tli_attention_decode_bf16.  One row per sequence.  head_dim a multiple of 64,
// at most 16 heads a kv head.
extern "C" int tli_qkv_attention_decode_bf16(
    const void* qkv, void* out, float* partial, void* k_cache, void* v_cache,
    const int* positions, const int* seq_of_row, const int* tables, int table_width, int page_size,
    int num_pages, int rows, int heads, int kv_heads, int head_dim,
    const float* q_norm_w, float q_eps, const float* k_norm_w, float k_eps,
    const float* cos_table, const float* sin_table, int write_cache,
    float scale, int window, int splits, int keys_per_split, const float* qkv_partial_sums, int qkv_parts,
    void* stream) {
    if (!qkv && !qkv_partial_sums) return tli_fail("attention_decode from raw projections: no projections");
    if (qkv_partial_sums && (qkv_parts < 1 || qkv_parts > 64 || ((uintptr_t)qkv_partial_sums & 15) || head_dim % 4))
        return tli_fail("attention_decode: %d planes of partial sums (1..64, 16-byte aligned)", qkv_parts);
    if ((cos_table == nullptr) != (sin_table == nullptr)) return tli_fail("attention_decode: cos without sin");
    const RawQkv raw{(const bf16_t*)qkv, q_norm_w, k_norm_w, cos_table, sin_table, q_eps, k_eps, write_cache,
                     qkv_partial_sums, qkv_parts, (size_t)rows * (heads + 2 * kv_heads) * head_dim};
    return launch_decode(nullptr, out, partial, k_cache, v_cache, positions, seq_of_row, tables, table_width,
                         page_size, num_pages, rows, heads, kv_heads, head_dim, scale, window, splits,
                         keys_per_split, &raw, stream);
}

// Rows of a sequence are contiguous and ascend in position; row_start has num_seqs+1 entries.
// direct = 1: every wave reads its keys and values straight from the cache (no LDS staging);
// 0: through LDS, tiles per wave by shape; 2, 3: through LDS with one, two tiles per wave.
static int launch_prefill(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* row_start,
    const int* seq_start, int num_seqs, int rows, const int* tables, int table_width, int page_size,
    int num_pages, int heads, int kv_heads, int head_dim, float scale, int window, int direct,
    const RawQkv* raw_in, void* stream) {
    if (rows <= 0 || num_seqs <= 0) return 0;
    if (check_common("attention_prefill", heads, kv_heads, head_dim, page_size, table_width, num_pages)) return 1;
    hipStream_t s = (hipStream_t)stream;
    const int group = heads / kv_heads, head_tiles = (group + 15) / 16;
    const int rq = group >= 16 ? 1 : 16 / group;
    const int shift = log2_exact(page_size);
    if (raw_in && (head_dim % 64 || page_size < 8 || direct == 1))
        return tli_fail("attention_prefill from raw projections: head_dim %d must be a multiple of 64, pages "
                        "of at least 8 (%d), through LDS", head_dim, page_size);
    const RawQkv raw = raw_in ? *raw_in : RawQkv{};
    if (page_size >= 8 && direct != 1) {
        // through LDS.  Two column tiles a wave when that still gives two workgroups for every
        // compute unit (long row blocks then come first); else one tile a wave.
        const long blocks1 = (rows + 4 * rq - 1) / (4 * rq) + num_seqs;
        const long blocks2 = (rows + 8 * rq - 1) / (8 * rq) + num_seqs;
        const long units = tli_compute_units();                   // 256 on MI355X
        bool two = head_dim <= 128 && blocks2 * kv_heads * head_tiles >= 2 * units;
        // Heads of 64 and 128, while the chip has room for every workgroup at once: the longest
        // workgroups decide the time, and two sets of waves a workgroup walk a workgroup's keys in
        // half the rounds (one workgroup a compute unit then: two tiles a wave where one tile would
        // make more than 256 workgroups).  Measured from 256 to 4,096 tokens, and portions of 512 to
        // 2,048 tokens behind up to 30,720: up to a third faster while all workgroups run at once
        // (256), a tenth faster up to 512 workgroups whose rows have no keys before them (the short
        // ones fill the second round), 3 to 15% slower there with keys before them (direct = 13 says
        // so: the lengths are on the device) and slower beyond.  Several sequences in a step have no such
        // long and short row blocks to share out: beyond two sequences the second round does not pay
        // either (8 sequences of 256 rows: 54 us in two sets, 42 us in one; 4 of 512: 58 and 50; one of
        // 2,000 beside 16 single rows: 93 and 77).
        const bool dma = head_dim == 64 || head_dim == 128;
        const long groups2 = (blocks2 - num_seqs) * kv_heads * head_tiles;
        bool sets = dma && groups2 <= (direct == 13 || num_seqs > 2 ? units : 2 * units);
        if (sets) two = (blocks1 - num_seqs) * kv_heads * head_tiles > units;
        // rows with keys before them are all about as long: two tiles a wave, which read the keys
        // once for both, already pay when one round of them fills the chip (1,536 rows behind
        // 6,656 keys: a fifth faster than one tile a wave)
        else if (dma && direct == 13 && groups2 > units) two = true;
        if (direct == 2) two = false;
        if (direct == 3 || (direct >= 4 && direct <= 7)) two = head_dim <= 128;
        if (direct == 8) two = false;
        if (head_dim == 112) two = false;                         // (two tiles of that size do not fit a wave's registers)
        if (direct == 12) two = true;                             // (measurements: 10 two sets, 11 one set, 12 two tiles in two sets)
        if (direct == 10 || direct == 12) sets = dma;
        if (direct == 11) sets = false;
        const int rows_per_block = 4 * rq * (two ? 2 : 1);
        const long blocks = (rows + rows_per_block - 1) / rows_per_block + num_seqs;   // upper bound
        if (blocks > 2147483647L) return tli_fail("attention_prefill: too many rows");
        int pair = two ? 3 : (blocks * kv_heads * head_tiles >= 4 * units ? 1 : 2);
        if (direct >= 4 && direct <= 7) pair = direct - 4;        // measurements: 4..7 force the pairing mode, two tiles
        if (direct == 8) pair = 3;                                // one tile, long blocks first
        if (sets && !(direct >= 4 && direct <= 7)) pair = 3;      // (one workgroup a compute unit: long blocks first)
        dim3 grid((unsigned)(pair == 1 ? (blocks + 1) / 2 : blocks), kv_heads * head_tiles);
        const int kb = head_dim <= 128 ? 64 : 32;
        // heads of 64 and 128: 32 keys a step copied straight into four LDS buffers
        const size_t lds = dma ? (size_t)4 * 2 * 32 * head_dim * sizeof(bf16_t)
                               : ((size_t)kb * (head_dim + 8) + (size_t)head_dim * (kb + 8)) * sizeof(bf16_t);
#define ARGS (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache, row_start, \
             seq_start, num_seqs, tables, table_width, page_size, shift, num_pages, heads, kv_heads
#define TAIL scale * LOG2E, window, rq
#define TAIL_LDS scale * LOG2E, window, rq, pair, raw
#define LDS_CALL(NJ, ND, CT, KB, DMA) attention_prefill_lds_kernel<NJ, ND, CT, KB, DMA><<<grid, 256, lds, s>>>(ARGS, TAIL_LDS)
        if (sets) {
            const size_t lds2 = 2 * lds;
#define SETS_CALL(NJ, ND, CT)                                                                            \
    {                                                                                                    \
        auto kernel = attention_prefill_lds_kernel<NJ, ND, CT, 32, true, 2>;                             \
        static bool allowed = false;                                                                     \
        if (lds2 > 65536 && !allowed) {                                                                  \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,     \
                                    (int)lds2) != hipSuccess)                                            \
                return tli_fail("attention_prefill: cannot have %zu bytes of LDS", lds2);                \
            allowed = true;                                                                              \
        }                                                                                                \
        kernel<<<grid, 512, lds2, s>>>(ARGS, TAIL_LDS);                                                  \
    }
            if (head_dim == 128 && two) SETS_CALL(4, 8, 2)
            else if (head_dim == 128) SETS_CALL(4, 8, 1)
            else if (two) SETS_CALL(2, 4, 2)
            else SETS_CALL(2, 4, 1)
#undef SETS_CALL
            return tli_check_launch("attention_prefill_lds");
        }
#define CALL(NJ, ND)                                                                                    \
    if ((ND == 4 || ND == 8) && two) LDS_CALL(((ND == 4 || ND == 8) ? ND / 2 : 2), ((ND == 4 || ND == 8) ? ND : 4), 2, 32, true); \
    else if (ND == 4 || ND == 8) LDS_CALL(((ND == 4 || ND == 8) ? ND / 2 : 2), ((ND == 4 || ND == 8) ? ND : 4), 1, 32, true); \
    else if (ND <= 8 && ND != 7 && two) LDS_CALL(NJ, ((ND <= 8 && ND != 4 && ND != 8 && ND != 7) ? ND : 1), 2, 64, false); \
    else if (ND <= 8) LDS_CALL(NJ, ((ND <= 8 && ND != 4 && ND != 8) ? ND : 1), 1, 64, false);           \
    else LDS_CALL(NJ, ND, 1, 32, false)
        DISPATCH_HEAD_DIM(CALL)
#undef CALL
#undef LDS_CALL
        return tli_check_launch("attention_prefill_lds");
    }
    {
        const int rows_per_block = 4 * rq;
        const long blocks = (rows + rows_per_block - 1) / rows_per_block + num_seqs;   // upper bound
        if (blocks > 2147483647L) return tli_fail("attention_prefill: too many rows");
        dim3 grid((unsigned)blocks, kv_heads * head_tiles);
#define CALL(NJ, ND) attention_prefill_kernel<NJ, ND, 1><<<grid, 256, 0, s>>>(ARGS, head_dim, TAIL)
        DISPATCH_HEAD_DIM(CALL)
#undef CALL
#undef ARGS
#undef TAIL
#undef TAIL_LDS
    }
    return tli_check_launch("attention_prefill");
}

extern "C" int tli_attention_prefill_bf16(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* row_start,
    const int* seq_start, int num_seqs, int rows, const int* tables, int table_width, int page_size,
    int num_pages, int heads, int kv_heads, int head_dim, float scale, int window, int direct,
    void* stream) {
    return launch_prefill(q, out, k_cache, v_cache, row_start, seq_start, num_seqs, rows, tables, table_width,
                          page_size, num_pages, heads, kv_heads, head_dim, scale, window, direct, nullptr, stream);
}

// The same with the queries taken from the raw projections qkv [rows][(heads + 2 kv_heads) * head_dim]
// (per-head norm if q_norm_w, rotation of the whole head if cos_table), the keys and values
// already in the cache.  head_dim a multiple of 64, pages of at least 8, direct != 1.
extern "C" int tli_qkv_attention_prefill_bf16(
    const void* qkv, void* out, const void* k_cache, const void* v_cache, const int* row_start,
    const int* seq_start, int num_seqs, int rows, const int* tables, int table_width, int page_size,
    int num_pages, int heads, int kv_heads, int head_dim, const float* q_norm_w, float q_eps,
    const float* cos_table, const float* sin_table, float scale, int window, int direct, void* stream) {
    if (!qkv) return tli_fail("attention_prefill from raw projections: no projections");
    if ((cos_table == nullptr) != (sin_table == nullptr)) return tli_fail("attention_prefill: cos without sin");
    const RawQkv raw{(const bf16_t*)qkv, q_norm_w, nullptr, cos_table, sin_table, q_eps, 0.f, 0};
    return launch_prefill(nullptr, out, k_cache, v_cache, row_start, seq_start, num_seqs, rows, tables,
                          table_width, page_size, num_pages, heads, kv_heads, head_dim, scale, window, direct,
                          &raw, stream);
}
