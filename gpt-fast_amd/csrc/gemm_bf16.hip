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

// Sum NV values (a power of two, at most 32) over the 64 lanes of a wave.  Halves of the
// value array are exchanged between lane halves, so the work is NV shuffles instead of
// 6 NV; afterwards lanes 2v and 2v+1 hold the total of value v in vals[0].
template <int NV>
__device__ __forceinline__ void wave_sum_many(float (&vals)[NV], int lane) {
    int off = 32;
#pragma unroll
    for (int half = NV / 2; half >= 1; half >>= 1) {
        const bool upper = (lane & off) != 0;
#pragma unroll
        for (int i = 0; i < half; ++i) {
            const float keep = upper ? vals[i + half] : vals[i];
            const float send = upper ? vals[i] : vals[i + half];
            vals[i] = keep + __shfl_xor(send, off, GFA_WAVE);
        }
        off >>= 1;
    }
    for (; off >= 1; off >>= 1) vals[0] += __shfl_xor(vals[0], off, GFA_WAVE);
}

// One workgroup = 4 waves; a wave owns WR = 4 rows of W (4 output columns, or 2 columns
// times {gate, up} in gate mode).  x is staged in shared memory in pieces of `kc` columns
// (all of K when it fits), so each 16 bytes of W meet their MT pieces of x from LDS.
template <int MT, int MODE>
__global__ __launch_bounds__(256) void skinny_dot_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M,
        int N, int K, int ldo, int gate_rows, int kc) {
    extern __shared__ uint4 xs[];                      // [MT][kc / 8]
    constexpr int WR = 4;
    constexpr int COLS = (MODE == 3) ? 2 : 4;
    const int lane = threadIdx.x & 63;
    const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * COLS;
    const bool active = n0 < N;
    const int kc8 = kc >> 3;

    const bf16_t* wrow[WR];
#pragma unroll
    for (int r = 0; r < WR; ++r) {
        int n = n0 + (MODE == 3 ? (r & 1) : r);
        if (n >= N) n = N - 1;                         // clamped rows are computed, not stored
        if (MODE == 3 && r >= 2) n += gate_rows;
        wrow[r] = w + (size_t)n * K;
    }
    float acc[WR * MT];
#pragma unroll
    for (int i = 0; i < WR * MT; ++i) acc[i] = 0.f;

    for (int k0 = 0; k0 < K; k0 += kc) {
        const int cur8 = ((K - k0 < kc) ? K - k0 : kc) >> 3;
        if (k0 > 0) __syncthreads();
        for (int idx = threadIdx.x; idx < MT * cur8; idx += 256) {
            const int m = idx / cur8, c = idx - m * cur8;
            xs[m * kc8 + c] = (m < M) ? *(const uint4*)(x + (size_t)m * K + k0 + c * 8)
                                      : make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
        if (active) {
            int c = lane;
            for (; c + 64 < cur8; c += 128) {          // two pieces of every row in flight
                Pack8 wa[WR], wb[WR];
#pragma unroll
                for (int r = 0; r < WR; ++r) {
                    wa[r].u = *(const uint4*)(wrow[r] + k0 + c * 8);
                    wb[r].u = *(const uint4*)(wrow[r] + k0 + (c + 64) * 8);
                }
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    Pack8 xa, xb;
                    xa.u = xs[m * kc8 + c];
                    xb.u = xs[m * kc8 + c + 64];
#pragma unroll
                    for (int r = 0; r < WR; ++r)
                        acc[r * MT + m] = dot8(wb[r], xb, dot8(wa[r], xa, acc[r * MT + m]));
                }
            }
            for (; c < cur8; c += 64) {
                Pack8 wa[WR];
#pragma unroll
                for (int r = 0; r < WR; ++r) wa[r].u = *(const uint4*)(wrow[r] + k0 + c * 8);
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    Pack8 xa;
                    xa.u = xs[m * kc8 + c];
#pragma unroll
                    for (int r = 0; r < WR; ++r) acc[r * MT + m] = dot8(wa[r], xa, acc[r * MT + m]);
                }
            }
        }
    }
    if (!active) return;
    wave_sum_many<WR * MT>(acc, lane);
    // the 64 / NV lanes of group v hold the total of value v = r * MT + m
    constexpr int GROUP = 64 / (WR * MT);
    float total = acc[0];
    float gate_v = 0.f;
    if (MODE == 3) gate_v = __shfl(total, (lane + 32) & 63, GFA_WAVE);   // value v + 2 MT
    const int v = lane / GROUP;
    const int r = v / MT, m = v - r * MT;
    if (lane % GROUP == 0 && r < COLS && m < M && n0 + r < N)
        skinny_store<MODE>(out, ldo, m, n0 + r, total, gate_v);
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
        constexpr int COLS = (MODE == 3) ? 2 : 4;
        const int blocks = (N + 4 * COLS - 1) / (4 * COLS);
        const int mt = mc == 1 ? 1 : mc == 2 ? 2 : mc <= 4 ? 4 : 8;
        int kc = (65536 / (mt * 2)) & ~511;            // 64 KiB of x per workgroup
        if (kc > K) kc = K;
        const size_t shmem = (size_t)mt * kc * sizeof(bf16_t);
        if (mt == 1)
            skinny_dot_kernel<1, MODE><<<blocks, 256, shmem, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows, kc);
        else if (mt == 2)
            skinny_dot_kernel<2, MODE><<<blocks, 256, shmem, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows, kc);
        else if (mt == 4)
            skinny_dot_kernel<4, MODE><<<blocks, 256, shmem, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows, kc);
        else
            skinny_dot_kernel<8, MODE><<<blocks, 256, shmem, stream>>>(xs, w, os, mc, N, K, ldo, gate_rows, kc);
    }
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Matrix-core version for 2..64 rows of x.  A workgroup owns 16 rows of W (16 + 16 in gate
// mode); its waves split K between them and each wave walks its share in pieces of
// 16 rows x 128 columns: coalesced 16-byte loads (256 contiguous bytes per row), through a
// wave-private padded LDS tile into the operand layout of v_mfma_f32_16x16x32_bf16 (lane
// l: row l % 16, columns 8 (l / 16) .. +7), against x fragments read from cache in the
// same layout.  The next piece is in flight while the current one is multiplied.  The
// waves' partial sums meet in LDS and are added in wave order, so the result does not
// depend on timing.  D layout: lane l holds rows 4 (l / 16) .. +3 of column l % 16.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

#define SM_SUBK 128
#define SM_PITCH (SM_SUBK * 2 + 16)          // bytes per staged row: 256 + pad against conflicts
#define SM_TILE (16 * SM_PITCH)

union Frag8 {
    uint4 u;
    bf16x8_t v;
};

template <int CT, int MODE>
__global__ __launch_bounds__(512) void skinny_mfma_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M,
        int N, int K, int ldo, int gate_rows) {
    constexpr int RT = (MODE == 3) ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, NW = blockDim.x >> 6;
    const int n0 = blockIdx.x * 16;
    char* stage = smem + (size_t)wave * (RT * SM_TILE);
    const int lrow = lane >> 4, lchunk = lane & 15;      // loading: row lrow + 4 j, 16-byte chunk
    const int fi = lane & 15, fg = lane >> 4;            // multiplying: row / column fi, k group fg
    const int T = (K + SM_SUBK - 1) / SM_SUBK;
    const int t_begin = (int)((long)wave * T / NW), t_end = (int)((long)(wave + 1) * T / NW);

    floatx4_t acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    const bf16_t* wsrc[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int n = n0 + lrow + 4 * j;
            if (n >= N) n = N - 1;                       // clamped rows are computed, not stored
            wsrc[rt][j] = w + (size_t)(n + rt * gate_rows) * K + lchunk * 8;
        }
    uint4 regs[RT][4];
    auto load_piece = [&](int t) {
        const int k = t * SM_SUBK + lchunk * 8;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                regs[rt][j] = (k < K) ? *(const uint4*)(wsrc[rt][j] + t * SM_SUBK)
                                      : make_uint4(0, 0, 0, 0);
    };
    if (t_begin < t_end) load_piece(t_begin);
    for (int t = t_begin; t < t_end; ++t) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *(uint4*)(stage + rt * SM_TILE + (lrow + 4 * j) * SM_PITCH + lchunk * 16) = regs[rt][j];
        if (t + 1 < t_end) load_piece(t + 1);
#pragma unroll
        for (int s = 0; s < SM_SUBK / 32; ++s) {
            const int kk = t * SM_SUBK + (s * 4 + fg) * 8;
            Frag8 b[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const int m = ct * 16 + fi;
                b[ct].u = (m < M && kk < K) ? *(const uint4*)(x + (size_t)m * K + kk)
                                            : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                Frag8 a;
                a.u = *(const uint4*)(stage + rt * SM_TILE + fi * SM_PITCH + (s * 4 + fg) * 16);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct)
                    acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b[ct].v, acc[rt][ct], 0, 0, 0);
            }
        }
    }
    if (NW > 1) {
        __syncthreads();                                 // staging is done; reuse it for the sums
        floatx4_t* red = (floatx4_t*)smem;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) red[((wave * RT + rt) * CT + ct) * 64 + lane] = acc[rt][ct];
        __syncthreads();
        if (wave != 0) return;
        for (int wv = 1; wv < NW; ++wv)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc[rt][ct] += red[((wv * RT + rt) * CT + ct) * 64 + lane];
    }
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = ct * 16 + fi;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + fg * 4 + j;
            if (n < N) skinny_store<MODE>(out, ldo, m, n, acc[0][ct][j], MODE == 3 ? acc[RT - 1][ct][j] : 0.f);
        }
    }
}

template <int MODE>
static int launch_skinny_mfma(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K,
                              int ldo, int gate_rows, hipStream_t stream) {
    constexpr int RT = (MODE == 3) ? 2 : 1;
    const int tiles = (N + 15) / 16;
    const int pieces = (K + SM_SUBK - 1) / SM_SUBK;
    const int ct = (M + 15) / 16;
    int nw = 1;                                          // waves per tile: aim at >= 2048 waves
    const int nw_max = (MODE == 3) ? 4 : 8;
    while (nw < nw_max && tiles * nw < 2048 && pieces >= 4 * nw) nw *= 2;
    size_t shmem = (size_t)nw * RT * SM_TILE;
    const size_t red = (size_t)nw * RT * ct * 64 * sizeof(floatx4_t);
    if (nw > 1 && red > shmem) shmem = red;
    switch (ct) {
        case 1: skinny_mfma_kernel<1, MODE><<<tiles, nw * 64, shmem, stream>>>(x, w, out, M, N, K, ldo, gate_rows); break;
        case 2: skinny_mfma_kernel<2, MODE><<<tiles, nw * 64, shmem, stream>>>(x, w, out, M, N, K, ldo, gate_rows); break;
        case 3: skinny_mfma_kernel<3, MODE><<<tiles, nw * 64, shmem, stream>>>(x, w, out, M, N, K, ldo, gate_rows); break;
        default: skinny_mfma_kernel<4, MODE><<<tiles, nw * 64, shmem, stream>>>(x, w, out, M, N, K, ldo, gate_rows); break;
    }
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_skinny_mfma_bf16(const void* x, const void* w, void* out, int M, int N, int K,
                                    int ldo, int mode, int gate_rows, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0) return (int)hipErrorInvalidValue;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    switch (mode) {
        case 0: return launch_skinny_mfma<0>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
        case 1: return launch_skinny_mfma<1>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
        case 2: return launch_skinny_mfma<2>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
        case 3: return launch_skinny_mfma<3>(xp, wp, out, M, N, K, ldo, gate_rows, stream);
    }
    return (int)hipErrorInvalidValue;
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
