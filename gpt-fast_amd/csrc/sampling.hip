// Choosing the next token from a row of float logits, one workgroup per row.
//
// greedy:  the index of the largest logit, the lowest index on ties.
// sample:  logits / max(temperature, 1e-5); entries below the k-th largest are dropped
//          (ties with it stay); softmax; then argmax(p_i / q_i) with q_i ~ Exp(1), which
//          draws index i with probability p_i (generate.py:40-57).  The noise q_i is a
//          counter-based function of (seed, row key, position, i), so a row's draw does
//          not depend on the other rows of the launch.
#include "common.h"
#include "sampling.h"
#include <mutex>
#include <stdio.h>

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
        uint32_t seed_lo, uint32_t seed_hi, const uint32_t* __restrict__ seed_dev,
        const int* __restrict__ row_keys, const int* __restrict__ positions, int position_offset,
        int* __restrict__ out, float* __restrict__ probs_out) {
    __shared__ ArgBest scratch[16];
    __shared__ float fscratch[16];
    __shared__ unsigned hist[256];
    __shared__ uint32_t sh_prefix;
    __shared__ int sh_remaining;
    if (seed_dev) {                  // the seed lives in device memory: a recorded launch
        seed_lo = seed_dev[0];       // can be replayed with another seed
        seed_hi = seed_dev[1];
    }
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

// `seed_dev`: null, or two 32-bit words in device memory (low, high) that replace `seed`.
extern "C" int gfa_sample(const float* logits, size_t row_stride, int n_rows, int V,
                          float temperature, int top_k, uint64_t seed, const uint32_t* seed_dev,
                          const int* row_keys, const int* positions, int position_offset, int* out,
                          float* probs_out, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    sample_kernel<<<n_rows, SMP_THREADS, 0, stream>>>(
        logits, row_stride, V, temperature, top_k, (uint32_t)(seed & 0xffffffffu),
        (uint32_t)(seed >> 32), seed_dev, row_keys, positions, position_offset, out, probs_out);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The same choices with a row spread over many workgroups, for large vocabularies: one
// workgroup per chunk of SPL_CHUNK logits, a handful of small launches whose partial
// results meet in a workspace.  Integer histograms are summed with atomics (the sum does
// not depend on the order); float partials are added in chunk order.  Workspace, per row:
//   int   hist[4][256]   (zero before the call; the kernel that reads a histogram clears it,
//                         so a workspace that was zero once stays usable call after call)
//   int   state[2] = {prefix key, remaining}
//   float pmax[NB], psum[NB], pbest_v[NB]            int   pbest_i[NB]
#define SPL_CHUNK 4096
#define SPL_THREADS 1024

struct SplitWs {
    unsigned* hist;      // [B][4][256]
    unsigned* state;     // [B][2]
    float* pmax;         // [B][NB]
    float* psum;         // [B][NB]
    float* pbest_v;      // [B][NB]
    int* pbest_i;        // [B][NB]
    int NB;
};

__device__ __forceinline__ void split_load(const float* row, int V, int chunk, float (&v)[4], int& i0) {
    i0 = chunk * SPL_CHUNK + threadIdx.x * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c) v[c] = (i0 + c < V) ? row[i0 + c] : __builtin_nanf("");
}

// pass 0..3 of the radix select: histogram of byte (3 - pass) of the keys that match the
// prefix chosen so far; pass 0 also records the chunk's maximum.
__global__ __launch_bounds__(SPL_THREADS) void split_hist_kernel(
        const float* __restrict__ logits, size_t row_stride, int V, int pass, int with_hist,
        SplitWs ws) {
    __shared__ unsigned hist[256];
    __shared__ float fscratch[16];
    const int chunk = blockIdx.x, b = blockIdx.y;
    float v[4];
    int i0;
    split_load(logits + b * row_stride, V, chunk, v, i0);
    if (pass == 0) {
        float m = -INFINITY;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (v[c] == v[c]) m = fmaxf(m, v[c]);
        m = block_max(m, fscratch);
        if (threadIdx.x == 0) ws.pmax[b * ws.NB + chunk] = m;
    }
    if (!with_hist) return;
    for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    const int shift = 24 - 8 * pass;
    const uint32_t mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    const uint32_t prefix = pass == 0 ? 0u : ws.state[b * 2];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        if (v[c] != v[c]) continue;
        const uint32_t key = order_key(v[c]);
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 256; i += blockDim.x)
        if (hist[i]) atomicAdd(&ws.hist[(b * 4 + pass) * 256 + i], hist[i]);
}

// after a histogram pass: the bin that holds the k-th largest key extends the prefix.
__global__ __launch_bounds__(256) void split_pick_kernel(int pass, int top_k, SplitWs ws) {
    __shared__ unsigned suffix[257];
    const int b = blockIdx.x, t = threadIdx.x;
    suffix[t] = ws.hist[(b * 4 + pass) * 256 + t];
    if (t == 0) suffix[256] = 0;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {          // suffix sums: suffix[t] = sum of bins >= t
        const unsigned add = (t + off < 256) ? suffix[t + off] : 0u;
        __syncthreads();
        suffix[t] += add;
        __syncthreads();
    }
    const unsigned rem = pass == 0 ? (unsigned)top_k : ws.state[b * 2 + 1];
    const unsigned prefix = pass == 0 ? 0u : ws.state[b * 2];
    ws.hist[(b * 4 + pass) * 256 + t] = 0;             // read above; zero again for the next call
    __syncthreads();
    if (suffix[t] >= rem && suffix[t + 1] < rem) {     // exactly one bin
        ws.state[b * 2] = prefix | ((unsigned)t << (24 - 8 * pass));
        ws.state[b * 2 + 1] = rem - suffix[t + 1];
    }
}

__device__ __forceinline__ float split_row_max(const SplitWs& ws, int b) {
    float m = -INFINITY;
    for (int c = 0; c < ws.NB; ++c) m = fmaxf(m, ws.pmax[b * ws.NB + c]);
    return m;
}

// partial sums of exp(v / t - max) over the kept entries of each chunk
__global__ __launch_bounds__(SPL_THREADS) void split_sum_kernel(
        const float* __restrict__ logits, size_t row_stride, int V, float t, int use_pivot,
        SplitWs ws) {
    __shared__ float fscratch[16];
    const int chunk = blockIdx.x, b = blockIdx.y;
    float v[4];
    int i0;
    split_load(logits + b * row_stride, V, chunk, v, i0);
    const uint32_t pivot = use_pivot ? ws.state[b * 2] : 0u;
    const float m = split_row_max(ws, b) / t;
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
        if (v[c] == v[c] && order_key(v[c]) >= pivot) sum += expf(v[c] / t - m);
    sum = block_sum(sum, fscratch);
    if (threadIdx.x == 0) ws.psum[b * ws.NB + chunk] = sum;
}

// probabilities, the exponential race, and each chunk's best candidate
__global__ __launch_bounds__(SPL_THREADS) void split_race_kernel(
        const float* __restrict__ logits, size_t row_stride, int V, float t, int use_pivot,
        uint32_t seed_lo, uint32_t seed_hi, const uint32_t* __restrict__ seed_dev,
        const int* __restrict__ row_keys, const int* __restrict__ positions, int position_offset,
        float* __restrict__ probs_out, SplitWs ws) {
    __shared__ ArgBest scratch[16];
    const int chunk = blockIdx.x, b = blockIdx.y;
    if (seed_dev) {
        seed_lo = seed_dev[0];
        seed_hi = seed_dev[1];
    }
    float v[4];
    int i0;
    split_load(logits + b * row_stride, V, chunk, v, i0);
    const uint32_t pivot = use_pivot ? ws.state[b * 2] : 0u;
    const float m = split_row_max(ws, b) / t;
    float total = 0.f;
    for (int c = 0; c < ws.NB; ++c) total += ws.psum[b * ws.NB + c];
    uint32_t ctr[4] = {(uint32_t)(i0 >> 2), (uint32_t)(positions ? positions[b] + position_offset
                                                                 : position_offset),
                       (uint32_t)row_keys[b], 0u};
    philox(ctr, seed_lo, seed_hi);
    ArgBest best = {0.f, -1};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        if (i0 + c >= V) break;
        float p = 0.f;
        if (v[c] == v[c] && order_key(v[c]) >= pivot) p = expf(v[c] / t - m) / total;
        if (probs_out) probs_out[(size_t)b * V + i0 + c] = p;
        if (p > 0.f) {
            ArgBest cand = {p / exp_noise(ctr[c]), i0 + c};
            best = better(best, cand);
        }
    }
    best = block_best(best, scratch);
    if (threadIdx.x == 0) {
        ws.pbest_v[b * ws.NB + chunk] = best.v;
        ws.pbest_i[b * ws.NB + chunk] = best.i;
    }
}

// each chunk's largest logit (greedy)
__global__ __launch_bounds__(SPL_THREADS) void split_argmax_kernel(
        const float* __restrict__ logits, size_t row_stride, int V, SplitWs ws) {
    __shared__ ArgBest scratch[16];
    const int chunk = blockIdx.x, b = blockIdx.y;
    float v[4];
    int i0;
    split_load(logits + b * row_stride, V, chunk, v, i0);
    ArgBest best = {0.f, -1};
#pragma unroll
    for (int c = 0; c < 4; ++c)
        if (v[c] == v[c]) {
            ArgBest cand = {v[c], i0 + c};
            best = better(best, cand);
        }
    best = block_best(best, scratch);
    if (threadIdx.x == 0) {
        ws.pbest_v[b * ws.NB + chunk] = best.v;
        ws.pbest_i[b * ws.NB + chunk] = best.i;
    }
}

__global__ __launch_bounds__(64) void split_final_kernel(int* __restrict__ out, SplitWs ws) {
    const int b = blockIdx.x;
    ArgBest best = {0.f, -1};
    for (int c = threadIdx.x; c < ws.NB; c += 64) {
        ArgBest cand = {ws.pbest_v[b * ws.NB + c], ws.pbest_i[b * ws.NB + c]};
        best = better(best, cand);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgBest y;
        y.v = __shfl_xor(best.v, o, 64);
        y.i = __shfl_xor(best.i, o, 64);
        best = better(best, y);
    }
    if (threadIdx.x == 0) out[b] = best.i < 0 ? 0 : best.i;
}

extern "C" size_t gfa_sample_split_workspace(int n_rows, int V) {
    const size_t nb = (V + SPL_CHUNK - 1) / SPL_CHUNK;
    return (size_t)n_rows * (4 * 256 + 2 + 4 * nb) * 4;
}

// temperature <= 0 means greedy.  `workspace` has gfa_sample_split_workspace bytes; its
// first n_rows * 1024 ints (the histograms) must be zero at the first call and are zero
// again when a call has run, so one workspace serves call after call on one stream.
// `seed_dev`: null, or two 32-bit words in device memory (low, high) that replace `seed`.
static int run_sample_split(const float* logits, size_t row_stride, int n_rows, int V,
                            float temperature, int top_k, uint64_t seed, const uint32_t* seed_dev,
                            const int* row_keys, const int* positions, int position_offset,
                            int* out, float* probs_out, void* workspace, hipStream_t stream) {
    SplitWs ws;
    ws.NB = (V + SPL_CHUNK - 1) / SPL_CHUNK;
    char* p = (char*)workspace;
    ws.hist = (unsigned*)p;      p += (size_t)n_rows * 4 * 256 * 4;
    ws.state = (unsigned*)p;     p += (size_t)n_rows * 2 * 4;
    ws.pmax = (float*)p;         p += (size_t)n_rows * ws.NB * 4;
    ws.psum = (float*)p;         p += (size_t)n_rows * ws.NB * 4;
    ws.pbest_v = (float*)p;      p += (size_t)n_rows * ws.NB * 4;
    ws.pbest_i = (int*)p;
    const dim3 grid(ws.NB, n_rows);
    if (temperature <= 0.f) {
        split_argmax_kernel<<<grid, SPL_THREADS, 0, stream>>>(logits, row_stride, V, ws);
        split_final_kernel<<<n_rows, 64, 0, stream>>>(out, ws);
        return GFA_LAUNCH_RESULT();
    }
    const float t = fmaxf(temperature, 1e-5f);
    const int use_pivot = (top_k > 0 && top_k < V) ? 1 : 0;
    for (int pass = 0; pass < (use_pivot ? 4 : 1); ++pass) {
        split_hist_kernel<<<grid, SPL_THREADS, 0, stream>>>(logits, row_stride, V, pass, use_pivot, ws);
        if (use_pivot) split_pick_kernel<<<n_rows, 256, 0, stream>>>(pass, top_k, ws);
    }
    split_sum_kernel<<<grid, SPL_THREADS, 0, stream>>>(logits, row_stride, V, t, use_pivot, ws);
    split_race_kernel<<<grid, SPL_THREADS, 0, stream>>>(
        logits, row_stride, V, t, use_pivot, (uint32_t)(seed & 0xffffffffu), (uint32_t)(seed >> 32),
        seed_dev, row_keys, positions, position_offset, probs_out, ws);
    split_final_kernel<<<n_rows, 64, 0, stream>>>(out, ws);
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_sample_split(const float* logits, size_t row_stride, int n_rows, int V,
                                float temperature, int top_k, uint64_t seed,
                                const uint32_t* seed_dev, const int* row_keys,
                                const int* positions, int position_offset, int* out,
                                float* probs_out, void* workspace, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (V <= 0 || !workspace) return (int)hipErrorInvalidValue;
    return run_sample_split(logits, row_stride, n_rows, V, temperature, top_k, seed, seed_dev,
                            row_keys, positions, position_offset, out, probs_out, workspace, stream);
}

// --------------------------------------------------------------------------------------
// The same without a workspace from the caller (declared and described in sampling.h).
// `scratch` is this library's copy of the array on each GPU; in host code its name is only
// a handle for hipGetSymbolAddress, never an address to pass on.
static __device__ __align__(256) unsigned char scratch[GFA_SAMPLE_STATIC_BYTES];

#define GFA_MAX_DEVICES 64
static void* scratch_of_device[GFA_MAX_DEVICES];          // the array's address on each GPU
static std::mutex scratch_lock;
static thread_local char last_error[256];

extern "C" const char* gfa_sampling_last_error(void) { return last_error; }

// The current GPU's array, looked up once per GPU with that GPU current.
static int scratch_here(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= GFA_MAX_DEVICES) {
        snprintf(last_error, sizeof last_error, "device %d: this library keeps scratch for devices 0..%d",
                 dev, GFA_MAX_DEVICES - 1);
        return (int)hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_of_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            snprintf(last_error, sizeof last_error, "hipGetSymbolAddress(scratch) on device %d: %s", dev,
                     hipGetErrorString(e));
            return e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
        }
        scratch_of_device[dev] = p;
    }
    *out = scratch_of_device[dev];
    return 0;
}

extern "C" int gfa_sampling_init(void) {
    void* p = nullptr;
    return scratch_here(&p);
}

__global__ __launch_bounds__(256) void clear_words_kernel(uint32_t* __restrict__ p, size_t n) {
    for (size_t i = blockIdx.x * (size_t)256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) p[i] = 0;
}

extern "C" int gfa_sample_split_static(const float* logits, size_t row_stride, int n_rows, int V,
                                       float temperature, int top_k, uint64_t seed,
                                       const uint32_t* seed_dev, const int* row_keys,
                                       const int* positions, int position_offset, int* out,
                                       float* probs_out, hipStream_t stream) {
    last_error[0] = 0;
    if (n_rows <= 0) return 0;
    if (V <= 0 || n_rows > GFA_SAMPLE_STATIC_MAX_ROWS || V > GFA_SAMPLE_STATIC_MAX_VOCAB ||
        gfa_sample_split_workspace(n_rows, V) > (size_t)GFA_SAMPLE_STATIC_BYTES) {
        snprintf(last_error, sizeof last_error,
                 "gfa_sample_split_static: %d rows of %d logits; its fixed scratch (%d bytes per GPU) "
                 "takes at most %d rows of at most %d logits", n_rows, V, (int)GFA_SAMPLE_STATIC_BYTES,
                 GFA_SAMPLE_STATIC_MAX_ROWS, GFA_SAMPLE_STATIC_MAX_VOCAB);
        return (int)hipErrorInvalidValue;
    }
    void* ws = nullptr;
    const int rc = scratch_here(&ws);
    if (rc != 0) return rc;
    const bool histograms = temperature > 0.f && top_k > 0 && top_k < V;
    if (histograms) {
        // whatever the last call left where this call's histograms lie (its own layout
        // depended on its sizes) goes; a kernel, not a memset, so that a recording replays it
        const size_t words = (size_t)n_rows * 4 * 256;
        clear_words_kernel<<<(unsigned)((words + 255) / 256), 256, 0, stream>>>((uint32_t*)ws, words);
    }
    return run_sample_split(logits, row_stride, n_rows, V, temperature, top_k, seed, seed_dev,
                            row_keys, positions, position_offset, out, probs_out, ws, stream);
}
