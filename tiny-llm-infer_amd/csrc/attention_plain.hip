// Plain attention over the paged cache: one workgroup per (head, row), any
// sizes, float32 or bfloat16 storage, float32 arithmetic.  This is the
// attention of the float32 path and the reference beside the tuned kernels.
//
// Row at position p, head h, kv head g = h / (heads / kv_heads):
//   s_t = (q_h . K_t,g) * scale   for t = lo..p,  lo = 0 or p - window + 1
//   out_h = sum_t softmax(s)_t V_t,g
// (kernels/src/paged_attention_cpu.cpp:16-69).  Keys are visited in tiles of
// 256 with a running maximum and sum, so no scratch grows with the context;
// the order of additions depends only on (lo, p), never on the batch.
#include "common.h"

#define AP_THREADS 256
#define AP_MAX_HEAD_DIM 512

template <typename T>
__global__ void attention_plain_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ seq_of_row, const int* __restrict__ tables, int table_width,
    int page_size, int num_pages, int heads, int kv_heads, int head_dim, float scale, int window) {
    __shared__ float q_s[AP_MAX_HEAD_DIM];
    __shared__ float p_s[AP_THREADS];
    __shared__ float red[16];
    const int row = blockIdx.x, head = blockIdx.y;
    const int tid = threadIdx.x;
    const int g = head / (heads / kv_heads);
    const int pos = positions[row];
    const int seq = seq_of_row[row];
    const int* table = tables + (size_t)seq * table_width;
    const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
    const size_t page_stride = (size_t)kv_heads * page_size * head_dim;

    const T* q_row = q + ((size_t)row * heads + head) * head_dim;
    for (int d = tid; d < head_dim; d += AP_THREADS) q_s[d] = to_f32(q_row[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc0 = 0.f, acc1 = 0.f;      // output elements tid and tid + 256
    for (int base = lo; base <= pos; base += AP_THREADS) {
        const int t = base + tid;
        float s = -INFINITY;
        if (t <= pos) {
            const int page = table[t / page_size];
            if (page >= 0 && page < num_pages) {
                const T* kp = k_cache + (size_t)page * page_stride +
                              ((size_t)g * page_size + (t % page_size)) * head_dim;
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot += q_s[d] * to_f32(kp[d]);
                s = dot * scale;
            }
        }
        const float tile_max = block_max(s, red);
        const float m_new = fmaxf(m, tile_max);
        const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float tile_sum = block_sum(p, red);
        l = l * corr + tile_sum;
        p_s[tid] = p;
        __syncthreads();
        const int count = min(AP_THREADS, pos - base + 1);
        for (int half = 0; half < 2; ++half) {
            const int d = tid + half * AP_THREADS;
            if (d >= head_dim) break;
            float a = (half == 0 ? acc0 : acc1) * corr;
            for (int j = 0; j < count; ++j) {
                const int tt = base + j;
                const int page = table[tt / page_size];
                if (page < 0 || page >= num_pages) continue;
                const T* vp = v_cache + (size_t)page * page_stride +
                              (size_t)g * page_size * head_dim + (tt % page_size);
                a += p_s[j] * to_f32(vp[(size_t)d * page_size]);
            }
            if (half == 0) acc0 = a; else acc1 = a;
        }
        m = m_new;
        __syncthreads();
    }
    T* o_row = out + ((size_t)row * heads + head) * head_dim;
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    if (tid < head_dim) from_f32(o_row + tid, acc0 * inv);
    if (tid + AP_THREADS < head_dim) from_f32(o_row + tid + AP_THREADS, acc1 * inv);
}

extern "C" int tli_attention_plain(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* positions,
    const int* seq_of_row, const int* tables, int table_width, int page_size, int num_pages,
    int rows, int heads, int kv_heads, int head_dim, float scale, int window, int dtype,
    void* stream) {
    if (rows <= 0) return 0;
    if (head_dim <= 0 || head_dim > AP_MAX_HEAD_DIM)
        return tli_fail("attention: head_dim %d is outside 1..%d", head_dim, AP_MAX_HEAD_DIM);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
        return tli_fail("attention: heads %d must be a multiple of kv heads %d", heads, kv_heads);
    if (heads > 65535) return tli_fail("attention: %d heads exceed the grid limit 65535", heads);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0)
        return tli_fail("attention: bad cache geometry");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(rows, heads);
    if (dtype == TLI_F32)
        attention_plain_kernel<float><<<grid, AP_THREADS, 0, s>>>(
            (const float*)q, (float*)out, (const float*)k_cache, (const float*)v_cache, positions,
            seq_of_row, tables, table_width, page_size, num_pages, heads, kv_heads, head_dim, scale, window);
    else if (dtype == TLI_BF16)
        attention_plain_kernel<bf16_t><<<grid, AP_THREADS, 0, s>>>(
            (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions,
            seq_of_row, tables, table_width, page_size, num_pages, heads, kv_heads, head_dim, scale, window);
    else
        return tli_fail("attention: unknown dtype %d", dtype);
    return tli_check_launch("attention_plain");
}
