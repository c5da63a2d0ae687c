// Sampling from float32 logits: arg-max, or Gumbel-max for a temperature.
//
// Greedy picks the largest logit, the lowest token id on ties
// (engine/src/llm_engine.cpp:81-85; kernels/src/sampling_kernel_cuda.cu:25-27).
// With temperature T > 1e-6 the score of token v is logit_v + T * (-log(-log u_v))
// (kernels/src/sampling_kernel_cuda.cu:50-54).  The reference draws u from
// Philox keyed by the thread index; here u_v is a hash of (seed, v) alone, so
// the draw does not depend on the launch shape or on the batch.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

#define SAMPLE_THREADS 1024

__host__ __device__ inline uint32_t tli_mix32(uint32_t h) {
    h ^= h >> 16; h *= 0x85ebca6bu; h ^= h >> 13; h *= 0xc2b2ae35u; h ^= h >> 16;
    return h;
}

// uniform in (0, 1): 23 bits of a hash of (seed, token) and a half, (k + 0.5) / 2^23.  Every such value is
// a float32 as it stands, the largest 1 - 2^-24.  (With 24 bits the largest, 16777215.5, rounds to 2^24:
// u = 1, a Gumbel value of +infinity, and that token drawn whatever its logit: one draw in a hundred over a
// vocabulary of 150 thousand.)
__host__ __device__ inline float tli_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t token) {
    uint32_t h = tli_mix32(token ^ 0x9e3779b9u);
    h = tli_mix32(h ^ seed_lo);
    h = tli_mix32(h + seed_hi * 0x85ebca6bu + 0x27d4eb2fu);
    return ((float)(h >> 9) + 0.5f) * (1.0f / 8388608.0f);
}

// f(token, logit) for the tokens t = threadIdx.x, threadIdx.x + blockDim.x, ..: eight loads are asked for
// before the first is used (one workgroup walks a whole row of 150 thousand logits: what bounds it is the
// wait for its loads).
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ l, int begin, int end, F&& f) {
    constexpr int U = 8;
    const int stride = blockDim.x;
    int t = begin + threadIdx.x;
    for (; t + (U - 1) * stride < end; t += U * stride) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = l[t + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) f(t + u * stride, v[u]);
    }
    for (; t < end; t += stride) f(t, l[t]);
}

#define TOPP_BINS 4096
#define TOPP_LEVELS 3

// The bin of logit v in a range that begins at `hi` and goes down: TOPP_BINS bins of 1 / scale each (what
// lies beyond the range falls into the first or the last bin).  Never smaller for a smaller v.
__device__ __forceinline__ int topp_bin(float hi, float scale, float v) {
    const float d = (hi - v) * scale;
    return d <= 0.f ? 0 : (d >= (float)(TOPP_BINS - 1) ? TOPP_BINS - 1 : (int)d);
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int vocab,
                              const float* __restrict__ temperatures,
                              const uint32_t* __restrict__ seeds, const float* __restrict__ top_p,
                              int* __restrict__ out) {
    __shared__ float best_v[SAMPLE_THREADS / TLI_WAVE];
    __shared__ int best_i[SAMPLE_THREADS / TLI_WAVE];
    __shared__ float red[16];
    __shared__ unsigned long long hist[TOPP_BINS], wave_sums[SAMPLE_THREADS / TLI_WAVE], crossing_above[1];
    __shared__ int crossing[1];
    const int row = blockIdx.x;
    const float* l = logits + (size_t)row * vocab;
    const float temp = temperatures ? temperatures[row] : 0.f;
    const bool draw = temp > 1.0e-6f;
    const uint32_t seed_lo = seeds ? seeds[2 * row] : 0u, seed_hi = seeds ? seeds[2 * row + 1] : 0u;

    // top-p (engine/src/llm_engine.cpp:118-141: tokens are taken in descending order until the running
    // sum of their weights exp((l - max)/T) reaches top_p * total): a token is kept if the weights of all
    // tokens strictly above it sum to less than top_p * total.  Found without sorting and in three passes
    // over the row: the weights go into a histogram over the logits' range, 4,096 bins from the top; the
    // bin in which the running sum reaches the threshold is cut into 4,096 bins again, and that one once
    // more.  Tokens above the last such bin are kept, tokens below it are not, and the tokens in it (logits
    // within 2^-36 of the row's range of each other) count as tied with its first, which is kept.  The
    // weights are summed as 64-bit integers (units of 2^-40), so the sums do not depend on the order in
    // which the threads add.
    float hi[TOPP_LEVELS], scale[TOPP_LEVELS];
    int star[TOPP_LEVELS];
    int levels = 0;
    if (draw && top_p && top_p[row] < 1.0f) {
        float mx = -INFINITY, mn = INFINITY;
        for_each_logit(l, 0, vocab, [&](int, float v) { mx = fmaxf(mx, v); mn = fminf(mn, v); });
        mx = block_max(mx, red);
        mn = -block_max(-mn, red);
        if (mx > mn) {
            const float inv_t = 1.0f / temp;
            unsigned long long above = 0, theta = 0;          // weights above the range in hand; the threshold
            hi[0] = mx;
            scale[0] = (float)TOPP_BINS / (mx - mn);
            for (int lev = 0; lev < TOPP_LEVELS; ++lev) {
                for (int b = threadIdx.x; b < TOPP_BINS; b += blockDim.x) hist[b] = 0;
                __syncthreads();
                for_each_logit(l, 0, vocab, [&](int, float v) {
                    bool in = true;
                    for (int k = 0; k < lev; ++k) in = in && topp_bin(hi[k], scale[k], v) == star[k];
                    if (in)
                        atomicAdd(&hist[topp_bin(hi[lev], scale[lev], v)],
                                  (unsigned long long)(expf((v - mx) * inv_t) * 1099511627776.0f));
                });
                __syncthreads();
                // running sums over the bins: a thread has TOPP_BINS / SAMPLE_THREADS bins in a row
                constexpr int MINE = TOPP_BINS / SAMPLE_THREADS;
                unsigned long long mine = 0;
                for (int j = 0; j < MINE; ++j) mine += hist[threadIdx.x * MINE + j];
                unsigned long long incl = mine;
                const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
                for (int off = 1; off < TLI_WAVE; off <<= 1) {
                    const unsigned long long up = __shfl_up(incl, off, TLI_WAVE);
                    if (lane >= off) incl += up;
                }
                if (lane == TLI_WAVE - 1) wave_sums[wave] = incl;
                if (threadIdx.x == 0) crossing[0] = -1;
                __syncthreads();
                unsigned long long before = above, all = 0;
                for (int w = 0; w < SAMPLE_THREADS / TLI_WAVE; ++w) {
                    if (w < wave) before += wave_sums[w];
                    all += wave_sums[w];
                }
                if (lev == 0) {
                    theta = (unsigned long long)((double)top_p[row] * (double)all);
                    if (theta < 1) theta = 1;
                }
                unsigned long long run = before + incl - mine;        // weights above this thread's first bin
                for (int j = 0; j < MINE; ++j) {
                    const unsigned long long h = hist[threadIdx.x * MINE + j];
                    if (run < theta && run + h >= theta) {             // (one bin of the row: the sums only grow)
                        crossing[0] = threadIdx.x * MINE + j;
                        crossing_above[0] = run;
                    }
                    run += h;
                }
                __syncthreads();
                if (crossing[0] < 0) break;                            // (cannot be: the last running sum is the total)
                star[lev] = crossing[0];
                above = crossing_above[0];
                levels = lev + 1;
                if (lev + 1 < TOPP_LEVELS) {
                    hi[lev + 1] = hi[lev] - (float)star[lev] / scale[lev];
                    scale[lev + 1] = scale[lev] * (float)TOPP_BINS;
                }
                __syncthreads();                                       // (everyone has read the crossing)
            }
        }
    }

    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for_each_logit(l, 0, vocab, [&](int t, float s) {
        bool kept = true;
        for (int k = 0; k < levels; ++k) {
            const int b = topp_bin(hi[k], scale[k], s);
            if (b != star[k]) {
                kept = b < star[k];
                break;
            }
        }
        if (!kept) return;
        if (draw) s += temp * -logf(-logf(tli_uniform(seed_lo, seed_hi, (uint32_t)t)));
        if (s > bv || (s == bv && t < bi)) { bv = s; bi = t; }
    });
    for (int off = TLI_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, TLI_WAVE);
        const int oi = __shfl_xor(bi, off, TLI_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    __syncthreads();
    if (lane == 0) { best_v[wave] = bv; best_i[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x / TLI_WAVE); ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
        out[row] = (bi == 0x7fffffff) ? 0 : bi;
    }
}

// Without top-p a row is cut into SAMPLE_CHUNKS pieces that one workgroup each scans
// (a single workgroup on 150 thousand logits is bound by latency); a second pass picks
// the best of the pieces.  The winner is the same: the highest score, lowest id on ties.
#define SAMPLE_CHUNKS 32

__global__ void sample_chunks_kernel(const float* __restrict__ logits, int vocab,
                                     const float* __restrict__ temperatures,
                                     const uint32_t* __restrict__ seeds, float* __restrict__ best_value,
                                     int* __restrict__ best_index) {
    __shared__ float bvs[256 / TLI_WAVE];
    __shared__ int bis[256 / TLI_WAVE];
    const int row = blockIdx.y, chunk = blockIdx.x;
    const float* l = logits + (size_t)row * vocab;
    const float temp = temperatures ? temperatures[row] : 0.f;
    const bool draw = temp > 1.0e-6f;
    const uint32_t lo = seeds ? seeds[2 * row] : 0u, hi = seeds ? seeds[2 * row + 1] : 0u;
    const int per = (vocab + SAMPLE_CHUNKS - 1) / SAMPLE_CHUNKS;
    const int begin = chunk * per, end = min(vocab, begin + per);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for_each_logit(l, begin, end, [&](int t, float s) {
        if (draw) s += temp * -logf(-logf(tli_uniform(lo, hi, (uint32_t)t)));
        if (s > bv || (s == bv && t < bi)) { bv = s; bi = t; }
    });
    for (int off = TLI_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, TLI_WAVE);
        const int oi = __shfl_xor(bi, off, TLI_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const int lane = threadIdx.x % TLI_WAVE, wave = threadIdx.x / TLI_WAVE;
    if (lane == 0) { bvs[wave] = bv; bis[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x / TLI_WAVE); ++w)
            if (bvs[w] > bv || (bvs[w] == bv && bis[w] < bi)) { bv = bvs[w]; bi = bis[w]; }
        best_value[row * SAMPLE_CHUNKS + chunk] = bv;
        best_index[row * SAMPLE_CHUNKS + chunk] = bi;
    }
}

__global__ void sample_pick_kernel(const float* __restrict__ best_value, const int* __restrict__ best_index,
                                   int* __restrict__ out) {
    const int row = blockIdx.x, lane = threadIdx.x;          // one wave
    float bv = lane < SAMPLE_CHUNKS ? best_value[row * SAMPLE_CHUNKS + lane] : -INFINITY;
    int bi = lane < SAMPLE_CHUNKS ? best_index[row * SAMPLE_CHUNKS + lane] : 0x7fffffff;
    for (int off = TLI_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, TLI_WAVE);
        const int oi = __shfl_xor(bi, off, TLI_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) out[row] = (bi == 0x7fffffff) ? 0 : bi;
}

// temperatures: float [rows] or null (greedy); seeds: uint32 [rows][2] (low, high word) or null;
// top_p: float [rows] or null (1 everywhere)
// scratch: rows * SAMPLE_CHUNKS * 8 bytes, used when top_p is null and the vocabulary is large
extern "C" int tli_sample(const float* logits, int rows, int vocab, const float* temperatures,
                          const uint32_t* seeds, const float* top_p, int* out, void* scratch, void* stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return tli_fail("sample: bad vocabulary size %d", vocab);
    if (temperatures && !seeds) return tli_fail("sample: temperatures need seeds");
    if (!top_p && scratch && vocab >= 8192 && rows <= 65535) {
        float* bv = (float*)scratch;
        int* bi = (int*)(bv + (size_t)rows * SAMPLE_CHUNKS);
        sample_chunks_kernel<<<dim3(SAMPLE_CHUNKS, rows), 256, 0, (hipStream_t)stream>>>(logits, vocab, temperatures,
                                                                                      seeds, bv, bi);
        if (tli_check_launch("sample_chunks")) return 1;
        sample_pick_kernel<<<rows, TLI_WAVE, 0, (hipStream_t)stream>>>(bv, bi, out);
        return tli_check_launch("sample_pick");
    }
    sample_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, vocab, temperatures, seeds,
                                                                     top_p, out);
    return tli_check_launch("sample");
}

extern "C" int tli_sample_scratch_bytes(int rows) { return rows * SAMPLE_CHUNKS * 8; }

// ---- the same sampling for callers that cannot allocate ---------------------------------
// The pieces' best scores and ids (what tli_sample takes as `scratch`) live in this array
// instead: TLI_SAMPLE_NO_ALLOC_MAX_ROWS * SAMPLE_CHUNKS * 8 bytes = 256 KiB on every GPU the
// library runs on, held until the process ends.  In host code the array's name is only a
// stand-in for the symbol; the address of each GPU's copy is asked for once, with that GPU
// current, and kept.  (No `used` attribute on it: that would keep the device symbol local
// to its code object, where the runtime cannot find it by name; the use in host code below
// is what keeps it.)
static __device__ __align__(256) unsigned char
    scratch[(size_t)TLI_SAMPLE_NO_ALLOC_MAX_ROWS * SAMPLE_CHUNKS * 8];

#define TLI_MAX_DEVICES 64
static void* g_scratch_of_device[TLI_MAX_DEVICES];
static std::mutex g_scratch_lock;

static int scratch_of_current_device(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return tli_fail("sample_no_alloc: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= TLI_MAX_DEVICES) return tli_fail("sample_no_alloc: device %d is beyond the %d this library keeps scratch for", dev, TLI_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_of_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return tli_fail("sample_no_alloc: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_of_device[dev] = p;
    }
    *ptr = g_scratch_of_device[dev];
    return 0;
}

extern "C" int tli_sample_no_alloc(const float* logits, int rows, int vocab, const float* temperatures,
                                   const uint32_t* seeds, const float* top_p, int* out, void* stream) {
    if (rows <= 0) return 0;
    if (rows > TLI_SAMPLE_NO_ALLOC_MAX_ROWS)
        return tli_fail("sample_no_alloc: %d rows, the scratch array of this entry point holds %d",
                        rows, TLI_SAMPLE_NO_ALLOC_MAX_ROWS);
    void* ptr = nullptr;
    if (scratch_of_current_device(&ptr)) return 1;
    // nothing in the array has to start at zero: the first pass writes every (row, piece)
    // entry that the second pass reads
    return tli_sample(logits, rows, vocab, temperatures, seeds, top_p, out, ptr, stream);
}

extern "C" int tli_sample_no_alloc_max_rows() { return TLI_SAMPLE_NO_ALLOC_MAX_ROWS; }

// Looks up the current device's copy of the array and launches nothing: for callers that
// record tli_sample_no_alloc into a HIP graph, so that the one query of the runtime (and the
// loading of this library's code on the device that may come with it) happens before the
// capture begins and not inside it.
extern "C" int tli_sample_no_alloc_prepare() {
    void* ptr = nullptr;
    return scratch_of_current_device(&ptr);
}

// the same draw on the host, for tests and for callers that hold logits there

extern "C" float tli_sample_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t token) {
    return tli_uniform(seed_lo, seed_hi, token);
}
