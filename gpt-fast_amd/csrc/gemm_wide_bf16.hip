// Matrix products with 17..64 rows of x (decoding a large batch): out = x W^T, x [M, K] and
// W [N, K] row-major bfloat16, float accumulation.
//
// The product is still bound by reading W once, but x (up to 64 x K) is now too large to be
// fetched from cache by every wave that needs it.  So the waves of a workgroup take
// different columns (16 rows of W each) over the SAME range of k and share x: a piece of x
// (all rows, 128 columns) is copied once per workgroup into LDS, double-buffered, and read
// from there by all waves in the operand layout of v_mfma_f32_16x16x32_bf16.  W goes, as in
// the few-row kernel, from coalesced 16-byte loads through a wave-private padded LDS tile
// into the same layout, two pieces ahead of the one being multiplied.
//
// A matrix with few columns (N = 4096: 32 workgroups of 128 columns) cannot fill the chip
// that way, so K is cut into slices, one workgroup per (column tile, slice).  Each writes its
// partial sums to a float workspace part [S, M, N]; a second kernel adds the slices in order
// (the result does not depend on timing) and applies what follows: the sum into the residual
// stream and the RMS norm after it, or the store of the plain result.
//
// Epilogues without slices (MODE): 0 store bfloat16, 1 store float, 2 add into a float
// matrix, 3 gate: out[m, n] = silu(x W[n]) * (x W[n + gate_rows]) in bfloat16 (model.py:227;
// a wave takes 8 gate rows and the 8 up rows that belong to them as one tile), 5 partial sums.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

#define WD_SUBK 128
#define WD_PITCH (WD_SUBK * 2 + 16)          // bytes per staged row: 256 + pad against conflicts
#define WD_TILE (16 * WD_PITCH)

union WFrag {
    uint4 u;
    bf16x8_t v;
};

__device__ __forceinline__ float wd_silu(float a) { return a / (1.f + expf(-a)); }

template <int CT, int MODE, int NW>
__global__ __launch_bounds__(NW * 64) void wide_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M,
        int N, int K, int ldo, int gate_rows, int pieces_per_slice) {
    constexpr int NT = NW * 64;
    constexpr int XBYTES = CT * 16 * WD_PITCH;             // one buffer of x: CT * 16 rows
    constexpr int XCHUNKS = CT * 16 * 16;                  // 16-byte pieces of an x buffer
    constexpr int XPER = (XCHUNKS + NT - 1) / NT;
    constexpr int COLS = (MODE == 3) ? 8 : 16;             // output columns per wave
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fi = lane & 15, fg = lane >> 4;              // multiplying: row / column fi, k group fg
    const int lrow = lane >> 4, lchunk = lane & 15;        // loading W: row lrow + 4 j, 16-byte chunk
    char* stage = smem + 2 * XBYTES + wave * WD_TILE;
    const int n0w = (blockIdx.x * NW + wave) * COLS;
    const int T = (K + WD_SUBK - 1) / WD_SUBK;
    const int t_begin = blockIdx.y * pieces_per_slice;
    const int t_end = (t_begin + pieces_per_slice < T) ? t_begin + pieces_per_slice : T;

    // a wave beyond the last column keeps loading x and meeting the barriers; its rows of W
    // are clamped and its results are not stored
    const bf16_t* wsrc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = lrow + 4 * j;
        int n = n0w + ((MODE == 3) ? (r & 7) : r);
        if (n >= N) n = N - 1;
        if (MODE == 3 && r >= 8) n += gate_rows;
        wsrc[j] = w + (size_t)n * K + lchunk * 8;
    }
    // this thread's pieces of an x buffer
    const bf16_t* xsrc[XPER];
    int xdst[XPER];
#pragma unroll
    for (int i = 0; i < XPER; ++i) {
        const int c = threadIdx.x + i * NT;
        const int row = c >> 4, chunk = c & 15;
        const bool ok = c < XCHUNKS && row < M;
        xsrc[i] = ok ? x + (size_t)row * K + chunk * 8 : nullptr;
        xdst[i] = (c < XCHUNKS) ? row * WD_PITCH + chunk * 16 : -1;
    }

    floatx4_t acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[ct] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    uint4 wa[4], wb[4], xr[XPER];
    auto load_w = [&](int t, uint4 (&regs)[4]) {
        const bool ok = t * WD_SUBK + lchunk * 8 < K;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            regs[j] = ok ? stream_load16(wsrc[j] + (size_t)t * WD_SUBK) : make_uint4(0, 0, 0, 0);
    };
    auto stage_w = [&](uint4 (&regs)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *(uint4*)(stage + (lrow + 4 * j) * WD_PITCH + lchunk * 16) = regs[j];
    };
    auto load_x = [&](int t) {
#pragma unroll
        for (int i = 0; i < XPER; ++i) {
            const int c = threadIdx.x + i * NT;
            const bool ok = xsrc[i] != nullptr && t * WD_SUBK + (c & 15) * 8 < K;
            xr[i] = ok ? *(const uint4*)(xsrc[i] + (size_t)t * WD_SUBK) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < XPER; ++i)
            if (xdst[i] >= 0) *(uint4*)(smem + buf * XBYTES + xdst[i]) = xr[i];
    };
    auto multiply = [&](int buf) {
        const char* xb = smem + buf * XBYTES;
#pragma unroll
        for (int s = 0; s < WD_SUBK / 32; ++s) {
            WFrag a;
            a.u = *(const uint4*)(stage + fi * WD_PITCH + (s * 4 + fg) * 16);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                WFrag b;
                b.u = *(const uint4*)(xb + (ct * 16 + fi) * WD_PITCH + (s * 4 + fg) * 16);
                acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[ct], 0, 0, 0);
            }
        }
    };

    if (t_begin < t_end) {
        load_x(t_begin);
        load_w(t_begin, wa);
        if (t_begin + 1 < t_end) load_w(t_begin + 1, wb);
        store_x(0);
        __syncthreads();
    }
    for (int t = t_begin; t < t_end; t += 2) {
        // piece t: x in buffer 0, W in wa
        if (t + 1 < t_end) load_x(t + 1);
        stage_w(wa);
        if (t + 2 < t_end) load_w(t + 2, wa);
        multiply(0);
        if (t + 1 < t_end) store_x(1);
        __syncthreads();
        if (t + 1 >= t_end) break;
        // piece t + 1: x in buffer 1, W in wb
        if (t + 2 < t_end) load_x(t + 2);
        stage_w(wb);
        if (t + 3 < t_end) load_w(t + 3, wb);
        multiply(1);
        if (t + 2 < t_end) store_x(0);
        __syncthreads();
    }

    // D layout: lane holds rows 4 fg .. 4 fg + 3 of the W tile (columns of out), x row fi
    if (n0w >= N) return;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = ct * 16 + fi;
        if (MODE == 3) {
            // rows 0..7 of the tile are gate columns, rows 8..15 their up columns: lanes of
            // groups 0, 1 hold the gates, groups 2, 3 the matching ups
            floatx4_t up;
#pragma unroll
            for (int j = 0; j < 4; ++j) up[j] = __shfl_xor(acc[ct][j], 32, GFA_WAVE);
            if (fg >= 2 || m >= M) continue;
            const int n = n0w + fg * 4;
            bf16_t* o = (bf16_t*)out + (size_t)m * ldo + n;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n + j < N) o[j] = float_to_bf16(wd_silu(acc[ct][j]) * up[j]);
            continue;
        }
        if (m >= M) continue;
        const int n = n0w + fg * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (n + j >= N) break;
            const float v = acc[ct][j];
            if (MODE == 0) {
                ((bf16_t*)out)[(size_t)m * ldo + n + j] = float_to_bf16(v);
            } else if (MODE == 1) {
                ((float*)out)[(size_t)m * ldo + n + j] = v;
            } else if (MODE == 2) {
                float* o = (float*)out + (size_t)m * ldo + n + j;
                *o = *o + v;
            } else {                                       // 5: this slice's partial sums
                ((float*)out)[((size_t)blockIdx.y * M + m) * N + n + j] = v;
            }
        }
    }
}

// Slices of K: enough workgroups to fill the chip, at least four pieces each.
static int wide_slices(int N, int K, int mode, int nw) {
    if (mode == 3) return 1;                               // the gate needs complete sums
    const int cols = nw * 16;
    const int tiles = (N + cols - 1) / cols;
    const int T = (K + WD_SUBK - 1) / WD_SUBK;
    int S = 1;
    while (tiles * S < 256 && T / (2 * S) >= 4) S *= 2;
    return S;
}

#ifndef WD_NW
#define WD_NW 8
#endif

// Number of slices the product [M, K] x [N, K] is cut into (1: no workspace needed).
extern "C" int gfa_wide_slices(int M, int N, int K, int mode) {
    (void)M;
    return wide_slices(N, K, mode, WD_NW);
}

template <int MODE>
static int launch_wide(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldo,
                       int gate_rows, int S, hipStream_t stream) {
    const int ct = (M + 15) / 16;
    constexpr int cols = WD_NW * ((MODE == 3) ? 8 : 16);
    const int tiles = (N + cols - 1) / cols;
    const int T = (K + WD_SUBK - 1) / WD_SUBK;
    const int per = (T + S - 1) / S;
    const dim3 grid(tiles, S);
#define GFA_LAUNCH_WIDE(CTV)                                                                      \
    do {                                                                                          \
        const size_t shmem = 2 * (size_t)(CTV * 16 * WD_PITCH) + (size_t)WD_NW * WD_TILE;         \
        static bool raised = false;                                                               \
        if (!raised) {                                                                            \
            hipFuncSetAttribute((const void*)wide_kernel<CTV, MODE, WD_NW>,                       \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);          \
            raised = true;                                                                        \
        }                                                                                         \
        wide_kernel<CTV, MODE, WD_NW><<<grid, WD_NW * 64, shmem, stream>>>(x, w, out, M, N, K,    \
                                                                           ldo, gate_rows, per);  \
    } while (0)
    switch (ct) {
        case 1: GFA_LAUNCH_WIDE(1); break;
        case 2: GFA_LAUNCH_WIDE(2); break;
        case 3: GFA_LAUNCH_WIDE(3); break;
        default: GFA_LAUNCH_WIDE(4); break;
    }
#undef GFA_LAUNCH_WIDE
    return GFA_LAUNCH_RESULT();
}

// x [M <= 64, K], w [N, K] (gate mode: [2 * N, K], gate_rows = N).  mode 0, 1, 2, 3: out
// [M, ldo] as above, one slice.  mode 5: out is the workspace [S, M, N] float with
// S = gfa_wide_slices(M, N, K, 5) (any mode but 3 gives the same number).
extern "C" int gfa_wide_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldo,
                             int mode, int gate_rows, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0) return (int)hipErrorInvalidValue;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    switch (mode) {
        case 0: return launch_wide<0>(xp, wp, out, M, N, K, ldo, gate_rows, 1, stream);
        case 1: return launch_wide<1>(xp, wp, out, M, N, K, ldo, gate_rows, 1, stream);
        case 2: return launch_wide<2>(xp, wp, out, M, N, K, ldo, gate_rows, 1, stream);
        case 3: return launch_wide<3>(xp, wp, out, M, N, K, ldo, gate_rows, 1, stream);
        case 5: return launch_wide<5>(xp, wp, out, M, N, K, ldo, gate_rows,
                                      wide_slices(N, K, 5, WD_NW), stream);
    }
    return (int)hipErrorInvalidValue;
}

// --------------------------------------------------------------------------------------
// Second kernels of a sliced product: the slices are added in order, s = 0 .. S - 1.

// out[m, n] = sum_s part[s, m, n], stored as bfloat16 or float
template <typename T>
__global__ __launch_bounds__(256) void wide_sum_store_kernel(const float* __restrict__ part, int S,
                                                             size_t slice, T* __restrict__ out,
                                                             size_t total) {
    const size_t e = (blockIdx.x * (size_t)256 + threadIdx.x) * 4;
    if (e >= total) return;
    if (e + 3 < total) {
        float4 a = *(const float4*)(part + e);
        for (int s = 1; s < S; ++s) {
            const float4 b = *(const float4*)(part + (size_t)s * slice + e);
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        store_from_float(out + e, a.x);
        store_from_float(out + e + 1, a.y);
        store_from_float(out + e + 2, a.z);
        store_from_float(out + e + 3, a.w);
    } else {
        for (size_t i = e; i < total; ++i) {
            float a = part[i];
            for (int s = 1; s < S; ++s) a += part[(size_t)s * slice + i];
            store_from_float(out + i, a);
        }
    }
}

extern "C" int gfa_wide_sum_store(const float* part, int S, int M, int N, void* out, int out_bf16,
                                  hipStream_t stream) {
    const size_t total = (size_t)M * N;
    if (total == 0 || S <= 0) return 0;
    if (N % 4 != 0) return (int)hipErrorInvalidValue;     // slices are read 16 bytes at a time
    const unsigned blocks = (unsigned)((total / 4 + 256) / 256);
    if (out_bf16)
        wide_sum_store_kernel<bf16_t><<<blocks, 256, 0, stream>>>(part, S, total, (bf16_t*)out, total);
    else
        wide_sum_store_kernel<float><<<blocks, 256, 0, stream>>>(part, S, total, (float*)out, total);
    return GFA_LAUNCH_RESULT();
}

// res[m, :] += sum_s part[s, m, :]; with norm_w also xn[m, :] = rmsnorm(res[m, :]) in
// bfloat16 (model.py:162-163 and 236-241): one workgroup per row, the row in registers.
template <int VPT>
__global__ __launch_bounds__(1024) void wide_sum_add_norm_kernel(
        float* __restrict__ res, const float* __restrict__ part, int S, size_t slice,
        const float* __restrict__ norm_w, bf16_t* __restrict__ xn, int dim, float eps) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    float4* rr = (float4*)(res + (size_t)m * dim);
    const int n4 = dim >> 2;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * 1024;
        v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (idx < n4) {
            float4 a = ((const float4*)(part + (size_t)m * dim))[idx];
            for (int s = 1; s < S; ++s) {
                const float4 b = ((const float4*)(part + (size_t)s * slice + (size_t)m * dim))[idx];
                a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
            }
            v[j] = rr[idx];
            v[j].x += a.x; v[j].y += a.y; v[j].z += a.z; v[j].w += a.w;
            rr[idx] = v[j];
        }
        ss = fmaf(v[j].x, v[j].x, ss);
        ss = fmaf(v[j].y, v[j].y, ss);
        ss = fmaf(v[j].z, v[j].z, ss);
        ss = fmaf(v[j].w, v[j].w, ss);
    }
    if (!norm_w) return;
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    uint2* o = (uint2*)(xn + (size_t)m * dim);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * 1024;
        if (idx < n4) {
            const float4 g = ((const float4*)norm_w)[idx];
            bf16_t e[4];
            e[0] = float_to_bf16(v[j].x * rs * g.x);
            e[1] = float_to_bf16(v[j].y * rs * g.y);
            e[2] = float_to_bf16(v[j].z * rs * g.z);
            e[3] = float_to_bf16(v[j].w * rs * g.w);
            o[idx] = make_uint2((unsigned)e[0] | ((unsigned)e[1] << 16),
                                (unsigned)e[2] | ((unsigned)e[3] << 16));
        }
    }
}

// dim: a multiple of 4, at most 16384.  norm_w and xn may be null (sum only).
extern "C" int gfa_wide_sum_add_norm(float* res, const float* part, int S, int M, int dim,
                                     const float* norm_w, void* xn, float eps, hipStream_t stream) {
    if (M <= 0 || dim <= 0 || S <= 0) return 0;
    if (dim % 4 != 0 || dim > 16384 || (norm_w != nullptr) != (xn != nullptr))
        return (int)hipErrorInvalidValue;
    const size_t slice = (size_t)M * dim;
    bf16_t* xp = (bf16_t*)xn;
    if (dim <= 4096) wide_sum_add_norm_kernel<1><<<M, 1024, 0, stream>>>(res, part, S, slice, norm_w, xp, dim, eps);
    else if (dim <= 8192) wide_sum_add_norm_kernel<2><<<M, 1024, 0, stream>>>(res, part, S, slice, norm_w, xp, dim, eps);
    else wide_sum_add_norm_kernel<4><<<M, 1024, 0, stream>>>(res, part, S, slice, norm_w, xp, dim, eps);
    return GFA_LAUNCH_RESULT();
}
