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

// Address of element (page, kv head, offset in page, 0) of one layer's page pool laid
// out as [n_pages, n_kv_heads, GFA_PAGE, head_dim].
__device__ __forceinline__ size_t page_row(int page, int kv_head, int offset, int n_kv_heads,
                                           int head_dim) {
    return (((size_t)page * n_kv_heads + kv_head) * GFA_PAGE + offset) * (size_t)head_dim;
}

// Values are kept transposed: one layer's pool is [n_pages, n_kv_heads, head_dim, GFA_PAGE],
// so that the keys of a page are contiguous for each element of the head.  The matrix-core
// attention reads its value operand (8 consecutive keys per lane) straight from this layout.
__device__ __forceinline__ size_t value_elem(int page, int kv_head, int d, int offset,
                                             int n_kv_heads, int head_dim) {
    return (((size_t)page * n_kv_heads + kv_head) * head_dim + d) * GFA_PAGE + offset;
}

#define GFA_LAUNCH_RESULT() ((int)hipGetLastError())
