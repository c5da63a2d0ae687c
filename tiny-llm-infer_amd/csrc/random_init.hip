// Seeded random weights: element e of tensor t of the model with seed s is a function of
// (s, t, e) alone, the same on the device, on the host and in a test's own version of it,
// bit for bit.  (The reference has no random-weights mode; its loader reads files only,
// model/src/qwen3_layers.cpp:76-147.)
//
// A 32-bit word is hashed from (s, t, e).  Its upper 16 bits pick an interval of the normal
// distribution's quantile function, given as a table of 65,537 float32 values q[i] = the
// quantile at i / 65536 (the two ends at a probability of 2^-18 from 0 and 1); its lower 16
// bits go from q[i] towards q[i + 1] in a straight line.  The result is mean + std * that.
// Every step is one float32 operation rounded on its own (nothing is fused into a multiply-add),
// so any processor with IEEE arithmetic gets the same bits; what remains of the normal
// distribution is cut at 4.5 standard deviations.
#include "common.h"
#include <thread>
#include <vector>

__host__ __device__ inline uint32_t rnd_mix32(uint32_t h) {
    h ^= h >> 16; h *= 0x85ebca6bu; h ^= h >> 13; h *= 0xc2b2ae35u; h ^= h >> 16;
    return h;
}

struct RandomKey { uint32_t k1, k2; };

// the part of the hash that is the same for every element of a tensor
static RandomKey random_key(uint32_t seed_lo, uint32_t seed_hi, uint32_t tensor) {
    RandomKey k;
    k.k1 = rnd_mix32(rnd_mix32(tensor ^ 0x9e3779b9u) ^ seed_lo);
    k.k2 = rnd_mix32(k.k1 + seed_hi * 0x85ebca6bu + 0x27d4eb2fu);
    return k;
}

__host__ __device__ inline uint32_t random_word(RandomKey k, uint64_t e) {
    uint32_t h = rnd_mix32((uint32_t)e ^ k.k1);
    return rnd_mix32(h + (uint32_t)(e >> 32) * 0x9e3779b1u + k.k2);
}

__global__ void random_normal_kernel(float* __restrict__ out, long long n, RandomKey key,
                                     const float* __restrict__ quantiles, float std, float mean) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
        const uint32_t w = random_word(key, (uint64_t)e);
        const float a = quantiles[w >> 16], b = quantiles[(w >> 16) + 1];
        const float frac = (float)(w & 0xffffu) * (1.0f / 65536.0f);         // exact
        // one rounding each, in this order
        const float z = __fadd_rn(a, __fmul_rn(__fsub_rn(b, a), frac));
        out[e] = __fadd_rn(mean, __fmul_rn(std, z));
    }
}

// the same on the host (volatile: the compiler may not fuse a product into the sum after it)
static void random_normal_host(float* out, long long begin, long long end, RandomKey key,
                               const float* quantiles, float std, float mean) {
    for (long long e = begin; e < end; ++e) {
        const uint32_t w = random_word(key, (uint64_t)e);
        const float a = quantiles[w >> 16], b = quantiles[(w >> 16) + 1];
        const float frac = (float)(w & 0xffffu) * (1.0f / 65536.0f);
        volatile float d = b - a;
        volatile float m = d * frac;
        volatile float z = a + m;
        volatile float s = std * z;
        out[e] = mean + s;
    }
}

// out: float32 [n], in device memory (on_device != 0; `quantiles` then too, 65,537 floats) or in
// host memory.  On the host the range is shared out over a few threads.
extern "C" int tli_random_normal(float* out, long long n, uint32_t seed_lo, uint32_t seed_hi, uint32_t tensor,
                                 const float* quantiles, float std, float mean, int on_device, void* stream) {
    if (n <= 0) return 0;
    if (!out || !quantiles) return tli_fail("random_normal: no output or no table of quantiles");
    const RandomKey key = random_key(seed_lo, seed_hi, tensor);
    if (on_device) {
        const long long blocks = (n + 255) / 256;
        random_normal_kernel<<<(unsigned)(blocks < 8192 ? blocks : 8192), 256, 0, (hipStream_t)stream>>>(
            out, n, key, quantiles, std, mean);
        return tli_check_launch("random_normal");
    }
    unsigned workers = std::thread::hardware_concurrency();
    workers = workers < 1 ? 1 : (workers > 16 ? 16 : workers);
    if (n < (1 << 20)) workers = 1;
    const long long piece = (n + workers - 1) / workers;
    std::vector<std::thread> threads;
    for (unsigned t = 1; t < workers; ++t) {
        const long long b = t * piece, e = b + piece < n ? b + piece : n;
        if (b < e) threads.emplace_back(random_normal_host, out, b, e, key, quantiles, std, mean);
    }
    random_normal_host(out, 0, piece < n ? piece : n, key, quantiles, std, mean);
    for (auto& th : threads) th.join();
    return 0;
}
