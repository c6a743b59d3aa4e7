// What this GPU reaches in the two resources the step is priced against, measured with
// kernels that do nothing else: bytes per second of a read stream and of a copy, and
// bfloat16 matrix-core flops per second.  bench.py prints them beside the datasheet peaks.
#include "common.h"

// Every workgroup reads a contiguous share of `src` in 16-byte pieces per lane, the same
// non-temporal loads the few-row products use for their weights, four in flight per lane.
__global__ __launch_bounds__(256) void read_stream_kernel(const uint4* __restrict__ src,
                                                          size_t n16, uint32_t* __restrict__ sink) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
    uint32_t acc = 0;
    size_t i = lo + threadIdx.x;
    for (; i + 768 < hi; i += 1024) {
        const uint4 a = stream_load16(src + i), b = stream_load16(src + i + 256);
        const uint4 c = stream_load16(src + i + 512), d = stream_load16(src + i + 768);
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w;
        acc ^= c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < hi; i += 256) {
        const uint4 a = stream_load16(src + i);
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u) sink[blockIdx.x] = acc;      // keeps the loads; almost never taken
}

__global__ __launch_bounds__(256) void copy_stream_kernel(uint4* __restrict__ dst,
                                                          const uint4* __restrict__ src, size_t n16) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
    for (size_t i = lo + threadIdx.x; i < hi; i += 256) dst[i] = stream_load16(src + i);
}

// bytes: a multiple of 16.  sink: at least `blocks` words.
extern "C" int gfa_read_stream(const void* src, size_t bytes, void* sink, int blocks,
                               hipStream_t stream) {
    if (bytes == 0 || bytes % 16 || blocks <= 0) return (int)hipErrorInvalidValue;
    read_stream_kernel<<<blocks, 256, 0, stream>>>((const uint4*)src, bytes / 16, (uint32_t*)sink);
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_copy_stream(void* dst, const void* src, size_t bytes, int blocks,
                               hipStream_t stream) {
    if (bytes == 0 || bytes % 16 || blocks <= 0) return (int)hipErrorInvalidValue;
    copy_stream_kernel<<<blocks, 256, 0, stream>>>((uint4*)dst, (const uint4*)src, bytes / 16);
    return GFA_LAUNCH_RESULT();
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

// Each wave issues `iters` rounds of eight independent v_mfma_f32_16x16x32_bf16 on operands
// that stay in registers: 8 * 16 * 16 * 32 * 2 flops per round and wave.
__global__ __launch_bounds__(256) void mfma_peak_kernel(float* __restrict__ out, int iters) {
    bf16x8_t a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 7));
        b[i] = (__bf16)(0.002f * (float)((threadIdx.x + 3 * i) & 7));
    }
    floatx4_t acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
    }
    floatx4_t s = acc[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) s += acc[j];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}

// out: blocks * 256 floats.  Flops of the launch: blocks * 4 waves * iters * 8 * 16384.
extern "C" int gfa_mfma_peak(float* out, int blocks, int iters, hipStream_t stream) {
    if (blocks <= 0 || iters <= 0) return (int)hipErrorInvalidValue;
    mfma_peak_kernel<<<blocks, 256, 0, stream>>>(out, iters);
    return GFA_LAUNCH_RESULT();
}
