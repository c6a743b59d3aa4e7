// Shared device helpers for the gfx950 kernels of this library.
//
// Conventions used by every kernel file:
//  * wavefronts are 64 lanes wide;
//  * activations are either float or bfloat16 (`bf16_t`, raw 16-bit storage); all
//    arithmetic on them is done in float;
//  * every entry point is `extern "C"`, takes raw device pointers and a stream, checks
//    nothing about pointer validity (the Python side checks shapes before the call) and
//    returns the hipError_t of the launch as an int.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define GFA_WAVE 64
#define GFA_PAGE 64            // tokens per cache page

typedef uint16_t bf16_t;      // storage of a bfloat16

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest, ties to even; NaN stays NaN (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    const __bf16 b = (__bf16)f;
    return __builtin_bit_cast(bf16_t, b);
}

// 16 bytes of a stream that is read once (the weights): a non-temporal load, so that the
// lines do not displace x, which every workgroup reads again and again, from the caches.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load16(const void* p) {
    const u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

template <typename T> __device__ __forceinline__ float load_as_float(const T* p);
template <> __device__ __forceinline__ float load_as_float<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_as_float<bf16_t>(const bf16_t* p) {
    return bf16_to_float(*p);
}
template <typename T> __device__ __forceinline__ void store_from_float(T* p, float v);
template <> __device__ __forceinline__ void store_from_float<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_from_float<bf16_t>(bf16_t* p, float v) {
    *p = float_to_bf16(v);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = GFA_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, GFA_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = GFA_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, GFA_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` is
// shared memory of at least 16 floats.  The order of additions depends only on the
// block size, so a row's result does not depend on what else is in the launch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (GFA_WAVE - 1), wave = threadIdx.x / GFA_WAVE;
    const int n_waves = (blockDim.x + GFA_WAVE - 1) / GFA_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < n_waves; ++w) t += scratch[w];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (GFA_WAVE - 1), wave = threadIdx.x / GFA_WAVE;
    const int n_waves = (blockDim.x + GFA_WAVE - 1) / GFA_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = scratch[0];
    for (int w = 1; w < n_waves; ++w) t = fmaxf(t, scratch[w]);
    return t;
}

// Layout of the cache.  One layer's pool of keys, and its pool of values, gives every
// (page, kv head) a region of GFA_PAGE * head_dim elements.  Inside a region the elements lie
// in the order in which the matrix-core attention reads its operands, so that a wave's load
// instruction covers whole, consecutive cache lines (with keys as rows of head_dim elements,
// the sixteen rows of an operand tile are sixteen lines, of which a load uses a quarter each:
// the single-token attention then spends more time on its loads than on anything else).
//
// Keys, head sizes that are multiples of 8: [32-key block][chunk of 8 dims][slot][8 dims].
// The 32 keys of a block fill two 16-row tiles of the score product; key 8 a + 4 t + b
// (a < 4, t < 2, b < 4) is row 4 a + b of tile t, slot 16 t + 4 a + b: the eight scores a lane
// receives then belong to eight consecutive keys, which is what the second product wants as
// its operand.  Other head sizes: rows [key][head_dim].
__device__ __forceinline__ size_t cache_region(int page, int kv_head, int n_kv_heads, int head_dim) {
    return ((size_t)page * n_kv_heads + kv_head) * GFA_PAGE * (size_t)head_dim;
}
__device__ __forceinline__ int key_slot(int key_in_block) {
    return ((key_in_block >> 2) & 1) * 16 + (key_in_block >> 3) * 4 + (key_in_block & 3);
}
__device__ __forceinline__ int key_offset(int key, int d, int head_dim) {
    if (head_dim % 8) return key * head_dim + d;
    return (key >> 5) * 32 * head_dim + (d >> 3) * 256 + key_slot(key & 31) * 8 + (d & 7);
}
__device__ __forceinline__ size_t key_elem(int page, int kv_head, int key, int d, int n_kv_heads,
                                           int head_dim) {
    return cache_region(page, kv_head, n_kv_heads, head_dim) + key_offset(key, d, head_dim);
}

// Values, head sizes that are multiples of 16: [16-dim tile][32-key block][8-key group][dim][8
// keys]: the operand of the second product for (tile, block) is 1 KB in lane order (lane
// 16 g + i: dim i of the tile, keys 8 g .. + 7 of the block).  Other head sizes: transposed
// rows [dim][GFA_PAGE].
__device__ __forceinline__ int value_offset(int d, int key, int head_dim) {
    if (head_dim % 16) return d * GFA_PAGE + key;
    return (d >> 4) * 1024 + (key >> 5) * 512 + ((key >> 3) & 3) * 128 + (d & 15) * 8 + (key & 7);
}
__device__ __forceinline__ size_t value_elem(int page, int kv_head, int d, int key, int n_kv_heads,
                                             int head_dim) {
    return cache_region(page, kv_head, n_kv_heads, head_dim) + value_offset(d, key, head_dim);
}

// Rows kept for a few-row product that reads them next ("chunked", pad = 4, 8, 16, 32 or 64
// rows, the least that holds them): [columns / 8][pad][8] instead of [rows][columns], so that the
// sixteen lanes which load one 16-byte chunk each of sixteen different rows read consecutive
// bytes (whole cache lines) instead of sixteen lines.  Element (m, n) of such rows:
__device__ __forceinline__ size_t chunked_elem(int m, int n, int pad) {
    return ((size_t)(n >> 3) * pad + m) * 8 + (n & 7);
}

#define GFA_LAUNCH_RESULT() ((int)hipGetLastError())
