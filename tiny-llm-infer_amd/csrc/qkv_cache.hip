// Per-head norm of q and k, rotation, and the write of k and v into the paged
// cache, in one pass over the fused projection output.
//
// For every row and head, in float32 (model/src/qwen3_paged_batch.cpp:160-227):
//   q, k:  x <- w * x / sqrt(mean(x^2) + eps)  over the head      (if a norm is given)
//          (x_i, x_{i+rd/2}) <- (x_i cos - x_{i+rd/2} sin, x_i sin + x_{i+rd/2} cos), i < rd/2
//                                                 (kernels/src/rope_kernel_cpu.cpp:156-179)
//   k -> keys[page = table[seq][pos / page_size]][kv head][pos % page_size][:]
//   v -> values[page][kv head][:][pos % page_size]      (values are kept transposed)
// q goes to its own [rows, heads*head_dim] buffer.  The cache layout differs from
// the reference's [page][slot][kv_dim] (kernels/src/paged_attention_cuda.cu:58-67):
// here the slots of one head in one page are contiguous.
#include "common.h"

#define QKV_MAX_HEAD_DIM 512
#define QKV_WAVES 4

template <typename T>
__global__ void qkv_to_cache_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_row,
    const int* __restrict__ tables, int table_width, int page_size, int num_pages,
    int heads, int kv_heads, int head_dim,
    const float* __restrict__ q_norm_w, float q_eps, const float* __restrict__ k_norm_w, float k_eps,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rotary_dim,
    int table_positions, int write_cache) {
    __shared__ float stage[QKV_WAVES][QKV_MAX_HEAD_DIM];
    const int row = blockIdx.x;
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    const int q_dim = heads * head_dim, kv_dim = kv_heads * head_dim;
    const int stride = q_dim + 2 * kv_dim;
    const int pos = positions[row];
    const T* src_row = qkv + (size_t)row * stride;

    // where this row's keys and values go
    size_t cache_base = 0, v_base = 0;
    bool can_write = false;
    if (write_cache) {
        const int seq = seq_of_row[row];
        const int page = tables[(size_t)seq * table_width + pos / page_size];
        can_write = page >= 0 && page < num_pages;
        cache_base = ((size_t)page * kv_heads * page_size + (size_t)(pos % page_size)) * head_dim;
        v_base = (size_t)page * kv_heads * head_dim * page_size + (size_t)(pos % page_size);
    }
    const int half = rotary_dim / 2;
    const float* cos_row = nullptr;
    const float* sin_row = nullptr;
    if (cos_table && pos >= 0 && pos < table_positions) {
        cos_row = cos_table + (size_t)pos * half;
        sin_row = sin_table + (size_t)pos * half;
    }

    float* x = stage[wave];
    // units 0..heads-1 are q heads, heads..heads+kv_heads-1 are k heads, then the v heads;
    // a workgroup takes QKV_WAVES consecutive units, one a wave
    const int h = blockIdx.y * QKV_WAVES + wave;
    if (h >= heads + 2 * kv_heads) return;
    if (h >= heads + kv_heads) {
        if (!can_write) return;
        const int g = h - heads - kv_heads;
        const T* vsrc = src_row + q_dim + kv_dim + (size_t)g * head_dim;
        for (int d = lane; d < head_dim; d += TLI_WAVE)
            v_cache[v_base + ((size_t)g * head_dim + d) * page_size] = cache_value(vsrc[d]);
        return;
    }
    {
        const bool is_q = h < heads;
        const T* src = src_row + (size_t)h * head_dim;     // q heads then k heads are contiguous
        const float* nw = is_q ? q_norm_w : k_norm_w;
        const float eps = is_q ? q_eps : k_eps;
        float ss = 0.f;
        for (int i = lane; i < head_dim; i += TLI_WAVE) {
            const float v = to_f32(src[i]);
            x[i] = v;
            ss += v * v;
        }
        if (nw) {
            ss = wave_sum(ss);
            const float scale = 1.0f / sqrtf(ss / (float)head_dim + eps);
            for (int i = lane; i < head_dim; i += TLI_WAVE) x[i] = nw[i] * x[i] * scale;
        }
        // lanes only touch the elements they wrote themselves until here; the
        // rotation reads a partner element written by another lane of this wave
        wave_lds_sync();
        T* dst;
        if (is_q) {
            dst = q_out + (size_t)row * q_dim + (size_t)h * head_dim;
        } else {
            if (!can_write) return;
            dst = k_cache + cache_base + (size_t)(h - heads) * page_size * head_dim;
        }
        for (int i = lane; i < head_dim; i += TLI_WAVE) {
            float v = x[i];
            if (cos_row && i < rotary_dim) {
                if (i < half) v = rotate_first_half(x[i], x[i + half], cos_row[i], sin_row[i]);
                else v = rotate_second_half(x[i], x[i - half], cos_row[i - half], sin_row[i - half]);
            }
            from_f32(dst + i, v);
        }
    }
}

// The same for head sizes that are multiples of 64 (EPL = head_dim / 64 elements a
// lane), without LDS: a lane holds EPL consecutive elements, so the first half of
// the head lies in lanes 0..31 and the rotation partner of lane l is lane l ^ 32.
// Needs rotary_dim == head_dim (or no rotation).  bfloat16 only.
template <int EPL>
__global__ void __launch_bounds__(QKV_WAVES * TLI_WAVE)
qkv_to_cache_wide_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache,
    bf16_t* __restrict__ v_cache, const int* __restrict__ positions, const int* __restrict__ seq_of_row,
    const int* __restrict__ tables, int table_width, int page_size, int num_pages,
    int heads, int kv_heads,
    const float* __restrict__ q_norm_w, float q_eps, const float* __restrict__ k_norm_w, float k_eps,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int table_positions,
    int write_cache, int first_unit, int end_unit) {
    constexpr int HD = 64 * EPL;
    const int row = blockIdx.x;
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    // units first_unit .. end_unit-1 of: q heads, k heads, v heads
    const int h = first_unit + blockIdx.y * QKV_WAVES + wave;
    if (h >= end_unit) return;
    const int q_dim = heads * HD, kv_dim = kv_heads * HD;
    const int pos = positions[row];
    const bf16_t* src = qkv + (size_t)row * (q_dim + 2 * kv_dim) + (size_t)h * HD + lane * EPL;
    const bool is_q = h < heads, is_v = h >= heads + kv_heads;

    int page = -1;
    if (write_cache && !is_q) {
        page = tables[(size_t)seq_of_row[row] * table_width + pos / page_size];
        if (page < 0 || page >= num_pages) return;
    } else if (!is_q) {
        return;                                       // keys and values of a read-only cache layer
    }
    // EPL consecutive elements of this lane
    float x[EPL];
    if (EPL == 1) {
        x[0] = bf16_to_f32(src[0]);
    } else if (EPL == 2) {
        const uint32_t u = *reinterpret_cast<const uint32_t*>(src);
        x[0] = bf16_to_f32((bf16_t)(u & 0xffffu));
        x[1 % EPL] = bf16_to_f32((bf16_t)(u >> 16));
    } else {
        const uint2 u = *reinterpret_cast<const uint2*>(src);
        x[0] = bf16_to_f32((bf16_t)(u.x & 0xffffu));
        x[1 % EPL] = bf16_to_f32((bf16_t)(u.x >> 16));
        x[2 % EPL] = bf16_to_f32((bf16_t)(u.y & 0xffffu));
        x[3 % EPL] = bf16_to_f32((bf16_t)(u.y >> 16));
    }
    if (is_v) {
        const int g = h - heads - kv_heads;
        bf16_t* dst = v_cache + ((size_t)page * kv_heads + g) * HD * page_size + (pos % page_size);
#pragma unroll
        for (int e = 0; e < EPL; ++e) dst[(size_t)(lane * EPL + e) * page_size] = cache_value(src[e]);
        return;
    }
    const float* nw = is_q ? q_norm_w : k_norm_w;
    if (nw) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) ss += x[e] * x[e];
        ss = wave_sum(ss);
        const float scale = 1.0f / sqrtf(ss / (float)HD + (is_q ? q_eps : k_eps));
#pragma unroll
        for (int e = 0; e < EPL; ++e) x[e] = nw[lane * EPL + e] * x[e] * scale;
    }
    if (cos_table && pos >= 0 && pos < table_positions) {
        const float* cr = cos_table + (size_t)pos * (HD / 2) + (lane % 32) * EPL;
        const float* sr = sin_table + (size_t)pos * (HD / 2) + (lane % 32) * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const float partner = __shfl_xor(x[e], 32, TLI_WAVE);
            x[e] = lane < 32 ? rotate_first_half(x[e], partner, cr[e], sr[e]) : rotate_second_half(x[e], partner, cr[e], sr[e]);
        }
    }
    bf16_t* dst = is_q ? q_out + (size_t)row * q_dim + (size_t)h * HD
                       : k_cache + (((size_t)page * kv_heads + (h - heads)) * page_size + (pos % page_size)) * HD;
    dst += lane * EPL;
    if (EPL == 1) {
        dst[0] = f32_to_bf16(x[0]);
    } else if (EPL == 2) {
        *reinterpret_cast<uint32_t*>(dst) = pack_bf16x2(x[0], x[1 % EPL]);
    } else {
        *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(x[0], x[1 % EPL]), pack_bf16x2(x[2 % EPL], x[3 % EPL]));
    }
}

// Which sequence and which of its groups a workgroup has: group `grp` of the step, where sequence
// s has the positions seq_start[s] .. + its rows, cut at multiples of G.  Every thread of the
// workgroup looks at one sequence (at a stride of the workgroup's size), the numbers of groups are
// summed up to each thread through LDS, and the thread whose sequence holds `grp` says so: a
// step of hundreds of sequences costs a workgroup a few rounds, not hundreds of dependent loads.
// Returns false if the step has fewer groups (the grid is an upper bound).  `found` is 4 ints of LDS.
template <int G>
__device__ __forceinline__ bool find_group(int grp, const int* __restrict__ row_start,
                                           const int* __restrict__ seq_start, int num_seqs, int* found,
                                           int* wave_totals, int& seq, int& start, int& first_row, int& n_rows,
                                           int& in_seq) {
    const int tid = threadIdx.x, lane = tid % TLI_WAVE, wave = tid / TLI_WAVE;
    const int waves = (blockDim.x + TLI_WAVE - 1) / TLI_WAVE;
    if (tid == 0) found[0] = -1;
    int base = 0;
    for (int s0 = 0; s0 < num_seqs; s0 += blockDim.x) {
        const int s = s0 + tid;
        int fr = 0, nr = 0, st = 0, g = 0;
        if (s < num_seqs) {
            fr = row_start[s];
            nr = row_start[s + 1] - fr;
            st = seq_start[s];
            g = nr > 0 ? (st + nr - 1) / G - st / G + 1 : 0;
        }
        int incl = g;                               // sum over the lanes up to this one
#pragma unroll
        for (int off = 1; off < TLI_WAVE; off <<= 1) {
            const int up = __shfl_up(incl, off, TLI_WAVE);
            if (lane >= off) incl += up;
        }
        __syncthreads();                            // (the totals of the round before have been read)
        if (lane == TLI_WAVE - 1) wave_totals[wave] = incl;
        __syncthreads();
        int before = base, total = 0;
        for (int w = 0; w < waves; ++w) {
            if (w < wave) before += wave_totals[w];
            total += wave_totals[w];
        }
        const int excl = before + incl - g;
        if (g > 0 && grp >= excl && grp < excl + g) {
            found[0] = s;
            found[1] = grp - excl;
        }
        base += total;
        __syncthreads();
        if (found[0] >= 0 || grp < base) break;     // (uniform: every thread reads the same words)
    }
    seq = found[0];
    if (seq < 0) return false;
    in_seq = found[1];
    first_row = row_start[seq];
    n_rows = row_start[seq + 1] - first_row;
    start = seq_start[seq];
    return true;
}

// The values of a step's rows into the cache, for steps that bring many rows a sequence: a
// workgroup takes up to G consecutive positions of one sequence that share a page and one kv
// head; a thread reads one dim of each of them (a wave reads whole rows) and writes them as one
// run of consecutive slots, where the kernels above write every (row, dim) as 2 bytes of its own.
// grid (groups upper bound, kv_heads).
template <int G>
__global__ void values_to_cache_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ v_cache, const int* __restrict__ row_start,
    const int* __restrict__ seq_start, int num_seqs, const int* __restrict__ tables, int table_width,
    int page_size, int num_pages, int heads, int kv_heads, int head_dim) {
    __shared__ int found[4], wave_totals[16];
    int seq, start, first_row, n_rows, grp;
    if (!find_group<G>(blockIdx.x, row_start, seq_start, num_seqs, found, wave_totals, seq, start, first_row, n_rows, grp))
        return;
    const int g0 = start / G + grp;
    const int p_lo = max(start, g0 * G), p_hi = min(start + n_rows, (g0 + 1) * G);
    const int n = p_hi - p_lo;
    const int page = tables[(size_t)seq * table_width + p_lo / page_size];
    if (page < 0 || page >= num_pages) return;
    const int slot0 = p_lo % page_size, kvh = blockIdx.y;
    const size_t stride = (size_t)(heads + 2 * kv_heads) * head_dim;
    const bf16_t* src = qkv + (size_t)(first_row + p_lo - start) * stride + (size_t)(heads + kv_heads + kvh) * head_dim;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        bf16_t vals[G];
#pragma unroll
        for (int j = 0; j < G; ++j) vals[j] = j < n ? cache_value(src[(size_t)j * stride + d]) : (bf16_t)0;
        bf16_t* dst = v_cache + (((size_t)page * kv_heads + kvh) * head_dim + d) * page_size + slot0;
        if (n == G) {               // a whole group: its slots start at a multiple of G
            uint32_t w[G / 2];
#pragma unroll
            for (int j = 0; j < G / 2; ++j) w[j] = (uint32_t)vals[2 * j] | ((uint32_t)vals[2 * j + 1] << 16);
            if (G == 16) {
                reinterpret_cast<uint4*>(dst)[0] = make_uint4(w[0], w[1], w[2], w[3]);
                reinterpret_cast<uint4*>(dst)[1] = make_uint4(w[4 % (G / 2)], w[5 % (G / 2)], w[6 % (G / 2)], w[7 % (G / 2)]);
            } else if (G == 8) {
                reinterpret_cast<uint4*>(dst)[0] = make_uint4(w[0], w[1], w[2], w[3]);
            } else {
#pragma unroll
                for (int j = 0; j < G / 2; ++j) reinterpret_cast<uint32_t*>(dst)[j] = w[j];
            }
        } else {
            for (int j = 0; j < n; ++j) dst[j] = vals[j];
        }
    }
}

// Keys and values of a step's rows into the cache in one pass, for steps that bring many rows a
// sequence and heads of 64, 128 or 256 (EPL = head_dim / 64 elements a lane): a workgroup takes
// up to G consecutive positions of one sequence that share a page, and one kv head.  Its four
// waves norm and rotate the keys of those positions, a row a wave at a time (as
// qkv_to_cache_wide_kernel does), and its threads then write the values as runs of slots (as
// values_to_cache_kernel does).  One launch instead of two: a kernel that follows another costs
// some 4 us on this chip however little it does.  grid (groups upper bound, kv_heads).
template <int EPL, int G>
__global__ void __launch_bounds__(QKV_WAVES * TLI_WAVE)
keys_values_to_cache_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    const int* __restrict__ row_start, const int* __restrict__ seq_start, int num_seqs,
    const int* __restrict__ tables, int table_width, int page_size, int num_pages, int heads, int kv_heads,
    const float* __restrict__ k_norm_w, float k_eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int table_positions) {
    constexpr int HD = 64 * EPL;
    __shared__ int found[4], wave_totals[16];
    int seq, start, first_row, n_rows, grp;
    if (!find_group<G>(blockIdx.x, row_start, seq_start, num_seqs, found, wave_totals, seq, start, first_row, n_rows, grp))
        return;
    const int g0 = start / G + grp;
    const int p_lo = max(start, g0 * G), p_hi = min(start + n_rows, (g0 + 1) * G);
    const int n = p_hi - p_lo;
    const int page = tables[(size_t)seq * table_width + p_lo / page_size];
    if (page < 0 || page >= num_pages) return;
    const int slot0 = p_lo % page_size, kvh = blockIdx.y;
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    const size_t stride = (size_t)(heads + 2 * kv_heads) * HD;
    const bf16_t* rows = qkv + (size_t)(first_row + p_lo - start) * stride;

    // keys: position p_lo + j by wave j % 4.  Everything a wave reads for its positions (their key rows, their
    // rows of the rotation tables) and for its share of the values is asked for before anything is
    // computed: the kernel is a chain of round trips to memory, and this makes one of what a loop over the
    // positions made two of for every position.
    constexpr int TURNS = G / QKV_WAVES;
    static_assert(G % QKV_WAVES == 0, "every wave takes the same number of positions");
    const bf16_t* ksrc = rows + (size_t)(heads + kvh) * HD + lane * EPL;
    bf16_t* kdst = k_cache + (((size_t)page * kv_heads + kvh) * page_size + slot0) * HD + lane * EPL;
    const bool rotate = cos_table != nullptr;
    uint2 kraw[TURNS];
    float cr[TURNS][EPL], sr[TURNS][EPL];
#pragma unroll
    for (int i = 0; i < TURNS; ++i) {
        const int j = min(wave + i * QKV_WAVES, n - 1);          // (a turn past the last position reads it again, and stores nothing)
        const bf16_t* src = ksrc + (size_t)j * stride;
        if (EPL == 1) kraw[i] = make_uint2((uint32_t)src[0], 0u);
        else if (EPL == 2) kraw[i] = make_uint2(*reinterpret_cast<const uint32_t*>(src), 0u);
        else kraw[i] = *reinterpret_cast<const uint2*>(src);
        const int pos = p_lo + j;
        const bool in_table = rotate && pos >= 0 && pos < table_positions;
        const size_t at = (size_t)(in_table ? pos : 0) * (HD / 2) + (lane % 32) * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            cr[i][e] = rotate ? cos_table[at + e] : 1.f;
            sr[i][e] = rotate ? sin_table[at + e] : 0.f;
        }
    }
    float knw[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) knw[e] = k_norm_w ? k_norm_w[lane * EPL + e] : 1.f;
    // values: one dim a thread, the positions as one run of slots
    const bf16_t* vsrc = rows + (size_t)(heads + kv_heads + kvh) * HD;
    const bool has_dim = (int)threadIdx.x < HD;                  // (HD <= 256 = the workgroup: a thread has one dim or none)
    bf16_t vals[G];
#pragma unroll
    for (int j = 0; j < G; ++j) vals[j] = has_dim && j < n ? cache_value(vsrc[(size_t)j * stride + threadIdx.x]) : (bf16_t)0;

#pragma unroll
    for (int i = 0; i < TURNS; ++i) {
        const int j = wave + i * QKV_WAVES;
        const int pos = p_lo + j;
        float x[EPL];
        x[0] = bf16_to_f32((bf16_t)(kraw[i].x & 0xffffu));
        if (EPL >= 2) x[1 % EPL] = bf16_to_f32((bf16_t)(kraw[i].x >> 16));
        if (EPL == 4) {
            x[2 % EPL] = bf16_to_f32((bf16_t)(kraw[i].y & 0xffffu));
            x[3 % EPL] = bf16_to_f32((bf16_t)(kraw[i].y >> 16));
        }
        if (k_norm_w) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) ss += x[e] * x[e];
            ss = wave_sum(ss);
            const float scale = 1.0f / sqrtf(ss / (float)HD + k_eps);
#pragma unroll
            for (int e = 0; e < EPL; ++e) x[e] = knw[e] * x[e] * scale;
        }
        if (rotate && pos >= 0 && pos < table_positions) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const float partner = __shfl_xor(x[e], 32, TLI_WAVE);
                x[e] = lane < 32 ? rotate_first_half(x[e], partner, cr[i][e], sr[i][e]) : rotate_second_half(x[e], partner, cr[i][e], sr[i][e]);
            }
        }
        if (j >= n) continue;
        bf16_t* dst = kdst + (size_t)j * HD;
        if (EPL == 1) {
            dst[0] = f32_to_bf16(x[0]);
        } else if (EPL == 2) {
            *reinterpret_cast<uint32_t*>(dst) = pack_bf16x2(x[0], x[1 % EPL]);
        } else {
            *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(x[0], x[1 % EPL]), pack_bf16x2(x[2 % EPL], x[3 % EPL]));
        }
    }

    if (has_dim) {
        const int d = threadIdx.x;
        bf16_t* dst = v_cache + (((size_t)page * kv_heads + kvh) * HD + d) * page_size + slot0;
        if (n == G) {               // a whole group: its slots start at a multiple of G
            uint32_t w[G / 2];
#pragma unroll
            for (int j = 0; j < G / 2; ++j) w[j] = (uint32_t)vals[2 * j] | ((uint32_t)vals[2 * j + 1] << 16);
            if (G == 16) {
                reinterpret_cast<uint4*>(dst)[0] = make_uint4(w[0], w[1], w[2], w[3]);
                reinterpret_cast<uint4*>(dst)[1] = make_uint4(w[4 % (G / 2)], w[5 % (G / 2)], w[6 % (G / 2)], w[7 % (G / 2)]);
            } else {
                reinterpret_cast<uint4*>(dst)[0] = make_uint4(w[0], w[1], w[2 % (G / 2)], w[3 % (G / 2)]);
            }
        } else {
            for (int j = 0; j < n; ++j) dst[j] = vals[j];
        }
    }
}

// Keys (normed, rotated) and values of the step's rows into the cache; q is left to the attention
// kernel that takes it from qkv itself.  bfloat16, head_dim 64, 128 or 256, the whole head rotated
// (or none of it), pages of 8 or more.
extern "C" int tli_keys_values_to_cache(
    const void* qkv, void* k_cache, void* v_cache, const int* row_start, const int* seq_start, int num_seqs,
    int rows, const int* tables, int table_width, int page_size, int num_pages, int heads, int kv_heads,
    int head_dim, const float* k_norm_w, float k_eps, const float* cos_table, const float* sin_table,
    int table_positions, void* stream) {
    if (rows <= 0 || num_seqs <= 0) return 0;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256)
        return tli_fail("keys_values_to_cache: head_dim %d, the kernel takes 64, 128 and 256", head_dim);
    if (heads <= 0 || kv_heads <= 0 || kv_heads > 65535) return tli_fail("keys_values_to_cache: bad head counts");
    if (page_size < 8 || (page_size & (page_size - 1)) || table_width <= 0 || num_pages <= 0)
        return tli_fail("keys_values_to_cache: bad cache geometry (pages of a power of two, at least 8)");
    if ((cos_table == nullptr) != (sin_table == nullptr)) return tli_fail("keys_values_to_cache: cos without sin");
    hipStream_t s = (hipStream_t)stream;
    const int G = page_size >= 16 ? 16 : 8;
    const long groups = (long)rows / G + 2L * num_seqs;           // upper bound
    if (groups > 2147483647L) return tli_fail("keys_values_to_cache: too many rows");
    dim3 grid((unsigned)groups, kv_heads);
#define KV(EPL, GG)                                                                                       \
    keys_values_to_cache_kernel<EPL, GG><<<grid, QKV_WAVES * TLI_WAVE, 0, s>>>(                           \
        (const bf16_t*)qkv, (bf16_t*)k_cache, (bf16_t*)v_cache, row_start, seq_start, num_seqs, tables,   \
        table_width, page_size, num_pages, heads, kv_heads, k_norm_w, k_eps, cos_table, sin_table,        \
        table_positions)
    if (head_dim == 64) { if (G == 16) KV(1, 16); else KV(1, 8); }
    else if (head_dim == 128) { if (G == 16) KV(2, 16); else KV(2, 8); }
    else { if (G == 16) KV(4, 16); else KV(4, 8); }
#undef KV
    return tli_check_launch("keys_values_to_cache");
}

// rows: the step's rows; row_start/seq_start as the prefill attention takes them.  bfloat16.
extern "C" int tli_values_to_cache(
    const void* qkv, void* v_cache, const int* row_start, const int* seq_start, int num_seqs, int rows,
    const int* tables, int table_width, int page_size, int num_pages, int heads, int kv_heads,
    int head_dim, void* stream) {
    if (rows <= 0 || num_seqs <= 0) return 0;
    if (head_dim <= 0 || heads <= 0 || kv_heads <= 0 || kv_heads > 65535) return tli_fail("values_to_cache: bad head sizes");
    if (page_size < 2 || (page_size & (page_size - 1)) || table_width <= 0 || num_pages <= 0)
        return tli_fail("values_to_cache: bad cache geometry (pages of a power of two, at least 2)");
    hipStream_t s = (hipStream_t)stream;
    const int G = page_size >= 16 ? 16 : page_size;
    const long groups = (long)rows / G + 2L * num_seqs;           // upper bound
    if (groups > 2147483647L) return tli_fail("values_to_cache: too many rows");
    dim3 grid((unsigned)groups, kv_heads);
    const int threads = head_dim <= 64 ? 64 : (head_dim <= 128 ? 128 : 256);
#define VALUES(GG)                                                                                       \
    values_to_cache_kernel<GG><<<grid, threads, 0, s>>>((const bf16_t*)qkv, (bf16_t*)v_cache, row_start, \
        seq_start, num_seqs, tables, table_width, page_size, num_pages, heads, kv_heads, head_dim)
    if (G == 16) VALUES(16);
    else if (G == 8) VALUES(8);
    else if (G == 4) VALUES(4);
    else VALUES(2);
#undef VALUES
    return tli_check_launch("values_to_cache");
}

// skip_values: the values are written by tli_values_to_cache instead.
extern "C" int tli_qkv_to_cache(
    const void* qkv, void* q_out, void* k_cache, void* v_cache, const int* positions,
    const int* seq_of_row, const int* tables, int table_width, int page_size, int num_pages,
    int rows, int heads, int kv_heads, int head_dim,
    const float* q_norm_w, float q_eps, const float* k_norm_w, float k_eps,
    const float* cos_table, const float* sin_table, int rotary_dim, int table_positions,
    int write_cache, int skip_values, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (head_dim <= 0 || head_dim > QKV_MAX_HEAD_DIM)
        return tli_fail("qkv_to_cache: head_dim %d is outside 1..%d", head_dim, QKV_MAX_HEAD_DIM);
    if (heads <= 0 || kv_heads <= 0) return tli_fail("qkv_to_cache: bad head counts");
    if (cos_table && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > head_dim))
        return tli_fail("qkv_to_cache: rotary_dim %d must be even and at most head_dim %d", rotary_dim, head_dim);
    if (write_cache && (page_size <= 0 || table_width <= 0 || num_pages <= 0))
        return tli_fail("qkv_to_cache: bad cache geometry");
    hipStream_t s = (hipStream_t)stream;
    const int threads = QKV_WAVES * TLI_WAVE;
    const int units = heads + 2 * kv_heads;
    if ((units + QKV_WAVES - 1) / QKV_WAVES > 65535) return tli_fail("qkv_to_cache: too many heads");
    dim3 grid(rows, (units + QKV_WAVES - 1) / QKV_WAVES);
    const bool wide = dtype == TLI_BF16 && head_dim % 64 == 0 && head_dim <= 256 && head_dim != 192 &&
                      (!cos_table || rotary_dim == head_dim);
    // without q_out only keys and values are done (the attention kernel takes q from qkv itself)
    const int first_unit = q_out ? 0 : heads, end_unit = heads + (skip_values ? 1 : 2) * kv_heads;
    if (!q_out || skip_values) {
        if (!wide) return tli_fail("qkv_to_cache: a part of the heads only for bfloat16 heads of 64, 128 or 256");
        if (!q_out && !write_cache) return 0;
        grid.y = (end_unit - first_unit + QKV_WAVES - 1) / QKV_WAVES;
    }
    if (wide) {
#define WIDE(EPL)                                                                                        \
    qkv_to_cache_wide_kernel<EPL><<<grid, threads, 0, s>>>(                                              \
        (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, positions, seq_of_row,   \
        tables, table_width, page_size, num_pages, heads, kv_heads, q_norm_w, q_eps, k_norm_w, k_eps,    \
        cos_table, sin_table, table_positions, write_cache, first_unit, end_unit)
        if (head_dim == 64) WIDE(1);
        else if (head_dim == 128) WIDE(2);
        else WIDE(4);
#undef WIDE
        return tli_check_launch("qkv_to_cache_wide");
    }
    if (dtype == TLI_F32)
        qkv_to_cache_kernel<float><<<grid, threads, 0, s>>>(
            (const float*)qkv, (float*)q_out, (float*)k_cache, (float*)v_cache, positions, seq_of_row,
            tables, table_width, page_size, num_pages, heads, kv_heads, head_dim, q_norm_w, q_eps,
            k_norm_w, k_eps, cos_table, sin_table, rotary_dim, table_positions, write_cache);
    else if (dtype == TLI_BF16)
        qkv_to_cache_kernel<bf16_t><<<grid, threads, 0, s>>>(
            (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, positions, seq_of_row,
            tables, table_width, page_size, num_pages, heads, kv_heads, head_dim, q_norm_w, q_eps,
            k_norm_w, k_eps, cos_table, sin_table, rotary_dim, table_positions, write_cache);
    else
        return tli_fail("qkv_to_cache: unknown dtype %d", dtype);
    return tli_check_launch("qkv_to_cache");
}
