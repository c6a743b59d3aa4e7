// Choosing the next token from a row of float logits, one workgroup per row.
//
// greedy:  the index of the largest logit, the lowest index on ties.
// sample:  logits / max(temperature, 1e-5); entries below the k-th largest are dropped
//          (ties with it stay); softmax; then argmax(p_i / q_i) with q_i ~ Exp(1), which
//          draws index i with probability p_i (generate.py:40-57).  The noise q_i is a
//          counter-based function of (seed, row key, position, i), so a row's draw does
//          not depend on the other rows of the launch.
#include "common.h"

#define SMP_THREADS 1024

struct ArgBest {
    float v;
    int i;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
    // larger value wins; equal values: lower index wins; index -1 (nothing) always loses
    if (b.i < 0) return a;
    if (a.i < 0) return b;
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

__device__ __forceinline__ ArgBest block_best(ArgBest x, ArgBest* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgBest y;
        y.v = __shfl_xor(x.v, o, 64);
        y.i = __shfl_xor(x.i, o, 64);
        x = better(x, y);
    }
    __syncthreads();
    if (lane == 0) scratch[wave] = x;
    __syncthreads();
    ArgBest r = scratch[0];
    const int n_waves = (blockDim.x + 63) >> 6;
    for (int w = 1; w < n_waves; ++w) r = better(r, scratch[w]);
    return r;
}

__global__ __launch_bounds__(SMP_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                              int* __restrict__ out, int V,
                                                              size_t row_stride) {
    __shared__ ArgBest scratch[16];
    const float* row = logits + blockIdx.x * row_stride;
    ArgBest best = {0.f, -1};
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v != v) continue;   // NaN never wins
        ArgBest c = {v, i};
        best = better(best, c);
    }
    best = block_best(best, scratch);
    if (threadIdx.x == 0) out[blockIdx.x] = best.i < 0 ? 0 : best.i;
}

extern "C" int gfa_argmax(const float* logits, int* out, int n_rows, int V, size_t row_stride,
                          hipStream_t stream) {
    if (n_rows <= 0) return 0;
    argmax_kernel<<<n_rows, SMP_THREADS, 0, stream>>>(logits, out, V, row_stride);
    return GFA_LAUNCH_RESULT();
}

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3").
__device__ __forceinline__ void philox(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
        const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
        c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// Exp(1) noise from 23 random bits: -log(u), u = (n + 1/2) / 2^23 lies strictly between
// 0 and 1 and is exact in float, so the noise is finite and positive.
__device__ __forceinline__ float exp_noise(uint32_t bits) {
    const float u = ((float)(bits >> 9) + 0.5f) * (1.0f / 8388608.0f);
    return -logf(u);
}

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(
        const float* __restrict__ logits, size_t row_stride, int V, float temperature, int top_k,
        uint32_t seed_lo, uint32_t seed_hi, const int* __restrict__ row_keys,
        const int* __restrict__ positions, int position_offset, int* __restrict__ out,
        float* __restrict__ probs_out) {
    __shared__ ArgBest scratch[16];
    __shared__ float fscratch[16];
    __shared__ unsigned hist[256];
    __shared__ uint32_t sh_prefix;
    __shared__ int sh_remaining;
    const int b = blockIdx.x;
    const float* row = logits + b * row_stride;
    const float t = fmaxf(temperature, 1e-5f);

    // k-th largest logit as an order key (0 = keep everything)
    uint32_t pivot_key = 0;
    if (top_k > 0 && top_k < V) {
        uint32_t prefix = 0, mask = 0;
        int remaining = top_k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
            __syncthreads();
            for (int i = threadIdx.x; i < V; i += blockDim.x) {
                const float v = row[i];
                if (v != v) continue;
                const uint32_t key = order_key(v);
                if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (threadIdx.x == 0) {
                int bin = 255, rem = remaining;
                for (; bin > 0; --bin) {
                    if ((int)hist[bin] >= rem) break;
                    rem -= (int)hist[bin];
                }
                sh_prefix = prefix | ((uint32_t)bin << shift);
                sh_remaining = rem;
            }
            __syncthreads();
            prefix = sh_prefix;
            remaining = sh_remaining;
            mask |= 255u << shift;
            __syncthreads();
        }
        pivot_key = prefix;
    }

    // maximum of the scaled logits that are kept
    float m = -INFINITY;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v != v || order_key(v) < pivot_key) continue;
        m = fmaxf(m, v / t);
    }
    m = block_max(m, fscratch);
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v != v || order_key(v) < pivot_key) continue;
        sum += expf(v / t - m);
    }
    sum = block_sum(sum, fscratch);

    const uint32_t key = (uint32_t)row_keys[b];
    const uint32_t pos = (uint32_t)(positions ? positions[b] + position_offset : position_offset);
    ArgBest best = {0.f, -1};
    for (int i4 = threadIdx.x * 4; i4 < V; i4 += blockDim.x * 4) {
        uint32_t c[4] = {(uint32_t)(i4 >> 2), pos, key, 0u};
        philox(c, seed_lo, seed_hi);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = i4 + j;
            if (i >= V) break;
            const float v = row[i];
            float p = 0.f;
            if (v == v && order_key(v) >= pivot_key) p = expf(v / t - m) / sum;
            if (probs_out) probs_out[(size_t)b * V + i] = p;
            if (p > 0.f) {
                ArgBest cand = {p / exp_noise(c[j]), i};
                best = better(best, cand);
            }
        }
    }
    best = block_best(best, scratch);
    if (threadIdx.x == 0) out[b] = best.i < 0 ? 0 : best.i;
}

extern "C" int gfa_sample(const float* logits, size_t row_stride, int n_rows, int V,
                          float temperature, int top_k, uint64_t seed, const int* row_keys,
                          const int* positions, int position_offset, int* out, float* probs_out,
                          hipStream_t stream) {
    if (n_rows <= 0) return 0;
    sample_kernel<<<n_rows, SMP_THREADS, 0, stream>>>(
        logits, row_stride, V, temperature, top_k, (uint32_t)(seed & 0xffffffffu),
        (uint32_t)(seed >> 32), row_keys, positions, position_offset, out, probs_out);
    return GFA_LAUNCH_RESULT();
}
