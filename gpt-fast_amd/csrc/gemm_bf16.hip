// Few-row matrix products with bfloat16 operands for decoding: out = x W^T with
// x [M, K] (M <= 64) and W [N, K], both row-major bfloat16, float accumulation.
//
// With few rows the product is bound by reading W once from HBM, so the kernels are
// organised around that stream: every wavefront owns a few rows of W and reads them
// front to back in 16-byte pieces per lane (1 KiB contiguous per wave and load), keeps
// one float accumulator per (row of W, row of x) and reduces over the lanes at the end.
// x is small and stays in cache.  Products use v_dot2_f32_bf16 (two multiply-adds per
// lane and instruction, float accumulate).
//
// Epilogues (MODE): 0 store bfloat16, 1 store float, 2 add into a float matrix (the
// residual stream), 3 gate: out[m, n] = silu(x W[n]) * (x W[n + gate_rows]) in bfloat16
// (the reference's feed-forward, model.py:227).
#include "common.h"

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;

union Pack8 {            // eight bfloat16 = one 16-byte load
    uint4 u;
    bf16x2_t h[4];
};

__device__ __forceinline__ float dot8(const Pack8& a, const Pack8& b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(a.h[i], b.h[i], acc, false);
    return acc;
}

__device__ __forceinline__ float silu(float a) { return a / (1.f + expf(-a)); }

template <int MODE>
__device__ __forceinline__ void skinny_store(void* out, int ldo, int m, int n, float v, float gate_v) {
    if (MODE == 0) {
        ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(v);
    } else if (MODE == 1) {
        ((float*)out)[(size_t)m * ldo + n] = v;
    } else if (MODE == 2) {
        float* o = (float*)out + (size_t)m * ldo + n;
        *o = *o + v;
    } else {
        ((bf16_t*)out)[(size_t)m * ldo + n] = float_to_bf16(silu(v) * gate_v);
    }
}

// R output columns per wave; in gate mode each column reads two rows of W.
template <int MT, int R, int MODE>
__global__ __launch_bounds__(256) void skinny_dot_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M,
        int N, int K, int ldo, int gate_rows) {
    constexpr int WR = (MODE == 3) ? 2 * R : R;        // rows of W per wave
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int n0 = wave * R;
    if (n0 >= N) return;

    const bf16_t* wrow[WR];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = (n0 + r < N) ? n0 + r : N - 1;    // clamp: duplicates are not stored
        wrow[r] = w + (size_t)n * K;
        if (MODE == 3) wrow[R + r] = w + (size_t)(n + gate_rows) * K;
    }
    float acc[WR][MT];
#pragma unroll
    for (int r = 0; r < WR; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;

#pragma unroll 2
    for (int k = lane * 8; k < K; k += 64 * 8) {
        Pack8 wv[WR], xv[MT];
#pragma unroll
        for (int r = 0; r < WR; ++r) wv[r].u = *(const uint4*)(wrow[r] + k);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < M) xv[m].u = *(const uint4*)(x + (size_t)m * K + k);
            else xv[m].u = make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < WR; ++r)
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[r][m] = dot8(wv[r], xv[m], acc[r][m]);
    }
#pragma unroll
    for (int r = 0; r < WR; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum(acc[r][m]);

    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (n0 + r >= N) continue;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m >= M) continue;
                skinny_store<MODE>(out, ldo, m, n0 + r, acc[r][m], MODE == 3 ? acc[R + r][m] : 0.f);
            }
        }
    }
}

// Any K (also not a multiple of 8): scalar loads, one wave per output column.
template <int MODE>
__global__ __launch_bounds__(256) void skinny_scalar_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M,
        int N, int K, int ldo, int gate_rows) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (n >= N) return;
    for (int m = 0; m < M; ++m) {
        float a = 0.f, b = 0.f;
        for (int k = lane; k < K; k += 64) {
            const float xv = bf16_to_float(x[(size_t)m * K + k]);
            a = fmaf(xv, bf16_to_float(w[(size_t)n * K + k]), a);
            if (MODE == 3) b = fmaf(xv, bf16_to_float(w[(size_t)(n + gate_rows) * K + k]), b);
        }
        a = wave_sum(a);
        if (MODE == 3) b = wave_sum(b);
        if (lane == 0) skinny_store<MODE>(out, ldo, m, n, a, b);
    }
}

template <int MODE>
static int launch_skinny(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K,
                         int ldo, int gate_rows, hipStream_t stream) {
    const size_t out_elem = (MODE == 0 || MODE == 3) ? sizeof(bf16_t) : sizeof(float);
    if (K % 8 != 0) {
        for (int m0 = 0; m0 < M; m0 += 16) {
            const int mc = (M - m0 < 16) ? M - m0 : 16;
            skinny_scalar_kernel<MODE><<<(N + 3) / 4, 256, 0, stream>>>(
                x + (size_t)m0 * K, w, (char*)out + (size_t)m0 * ldo * out_elem, mc, N, K, ldo,
                gate_rows);
        }
        return GFA_LAUNCH_RESULT();
    }
    for (int m0 = 0; m0 < M; m0 += 8) {
        const int mc = (M - m0 < 8) ? M - m0 : 8;
        const bf16_t* xs = x + (size_t)m0 * K;
        void* os = (char*)out + (size_t)m0 * ldo * out_elem;
        constexpr int R = (MODE == 3) ? 1 : 2;
        const int waves = (N + R - 1) / R;
        const int blocks = (waves + 3) / 4;
        if (mc == 1)
            skinny_dot_kernel<1, R, MODE><<<blocks, 256, 0, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows);
        else if (mc == 2)
            skinny_dot_kernel<2, R, MODE><<<blocks, 256, 0, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows);
        else if (mc <= 4)
            skinny_dot_kernel<4, R, MODE><<<blocks, 256, 0, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows);
        else
            skinny_dot_kernel<8, R, MODE><<<blocks, 256, 0, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows);
    }
    return GFA_LAUNCH_RESULT();
}

// x [M, K], w [N, K] (gate mode: [2 * N, K], gate_rows = N), out [M, ldo].
extern "C" int gfa_skinny_bf16(const void* x, const void* w, void* out, int M, int N, int K,
                               int ldo, int mode, int gate_rows, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0) return (int)hipErrorInvalidValue;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    switch (mode) {
        case 0: return launch_skinny<0>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
        case 1: return launch_skinny<1>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
        case 2: return launch_skinny<2>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
        case 3: return launch_skinny<3>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
    }
    return (int)hipErrorInvalidValue;
}
