// Plain kernels for every op of a decoder step.
//
// These are the reference kernels of the library: simple, one workgroup per row or per
// (token, head), all arithmetic in float.  The float32 engine runs on them alone; the
// bfloat16 engine uses them where no faster kernel exists, and the faster kernels are
// tested against them.  In each kernel the order of floating-point additions that
// produce one output element depends only on that element's own inputs (its row, its
// position), never on the number of rows or on the other sequences of the launch, so a
// float32 result is the same however the tokens were cut into steps or batched.
#include "common.h"

// --------------------------------------------------------------------------------------
// embedding gather: out[n, :] = float(table[tokens[n], :])          (model.py:140)
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ out, int dim) {
    const int n = blockIdx.x;
    const T* row = table + (size_t)tokens[n] * dim;
    float* o = out + (size_t)n * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] = load_as_float(row + d);
}

extern "C" int gfa_embed(const void* table, int table_bf16, const int* tokens, float* out,
                         int n_tokens, int dim, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (table_bf16)
        embed_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)table, tokens, out, dim);
    else
        embed_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, tokens, out, dim);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// RMS norm: out[i, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w[:],  r = rows ? rows[i] : i
// (model.py:236-241; statistics in float, one rounding at the store)
template <typename T>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               const int* __restrict__ rows, T* __restrict__ out, int dim,
                               float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    const float* xr = x + (size_t)r * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = xr[d];
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    T* o = out + (size_t)i * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) store_from_float(o + d, xr[d] * rs * w[d]);
}

// The same for rows of up to 1024 * VPT elements (a multiple of 4): the row is read once
// with 16-byte loads, kept in registers between the sum and the scaling.
template <typename T, int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_vec_kernel(
        const float* __restrict__ x, const float* __restrict__ w, const int* __restrict__ rows,
        T* __restrict__ out, int dim, float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    const float4* xr = (const float4*)(x + (size_t)r * dim);
    const float4* w4 = (const float4*)w;
    const int n4 = dim >> 2;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        v[j] = idx < n4 ? xr[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
        ss = fmaf(v[j].x, v[j].x, ss);
        ss = fmaf(v[j].y, v[j].y, ss);
        ss = fmaf(v[j].z, v[j].z, ss);
        ss = fmaf(v[j].w, v[j].w, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    T* o = out + (size_t)i * dim;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = w4[idx];
            store_from_float(o + 4 * idx + 0, v[j].x * rs * g.x);
            store_from_float(o + 4 * idx + 1, v[j].y * rs * g.y);
            store_from_float(o + 4 * idx + 2, v[j].z * rs * g.z);
            store_from_float(o + 4 * idx + 3, v[j].w * rs * g.w);
        }
    }
}

template <typename T>
static bool launch_rmsnorm_vec(const float* x, const float* w, const int* rows, T* out, int n_rows,
                               int dim, float eps, hipStream_t stream) {
    if (dim % 4 != 0 || dim > 8192) return false;
    // one float4 per thread where the row allows it: the kernel is a chain of latencies
    if (dim <= 1024) rmsnorm_vec_kernel<T, 1, 256><<<n_rows, 256, 0, stream>>>(x, w, rows, out, dim, eps);
    else if (dim <= 4096) rmsnorm_vec_kernel<T, 1, 1024><<<n_rows, 1024, 0, stream>>>(x, w, rows, out, dim, eps);
    else rmsnorm_vec_kernel<T, 2, 1024><<<n_rows, 1024, 0, stream>>>(x, w, rows, out, dim, eps);
    return true;
}

extern "C" int gfa_rmsnorm(const float* x, const float* w, const int* rows, void* out,
                           int out_bf16, int n_rows, int dim, float eps, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (out_bf16 ? launch_rmsnorm_vec<bf16_t>(x, w, rows, (bf16_t*)out, n_rows, dim, eps, stream)
                 : launch_rmsnorm_vec<float>(x, w, rows, (float*)out, n_rows, dim, eps, stream))
        return GFA_LAUNCH_RESULT();
    if (out_bf16)
        rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, w, rows, (bf16_t*)out, dim, eps);
    else
        rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>(x, w, rows, (float*)out, dim, eps);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The sum that completes a block and the norm that opens the next, one pass over each row:
// res[i, :] += float(y[i, :]);  out[i, :] = rmsnorm(res[i, :]) in bfloat16
// (model.py:162-163 followed by 236-241; the sum and the statistics in float)
__global__ void add_rmsnorm_kernel(float* __restrict__ res, const bf16_t* __restrict__ y,
                                   const float* __restrict__ w, bf16_t* __restrict__ out, int dim,
                                   float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    float* xr = res + (size_t)i * dim;
    const bf16_t* yr = y + (size_t)i * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = xr[d] + bf16_to_float(yr[d]);
        xr[d] = v;                                       // read back by this thread only
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    bf16_t* o = out + (size_t)i * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) store_from_float(o + d, xr[d] * rs * w[d]);
}

// rows of up to 1024 * VPT elements (a multiple of 4), kept in registers
template <int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_vec_kernel(
        float* __restrict__ res, const bf16_t* __restrict__ y, const float* __restrict__ w,
        bf16_t* __restrict__ out, int dim, float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    float4* xr = (float4*)(res + (size_t)i * dim);
    const uint2* yr = (const uint2*)(y + (size_t)i * dim);
    const float4* w4 = (const float4*)w;
    const int n4 = dim >> 2;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (idx < n4) {
            v[j] = xr[idx];
            const uint2 a = yr[idx];
            v[j].x += __uint_as_float(a.x << 16);
            v[j].y += __uint_as_float(a.x & 0xffff0000u);
            v[j].z += __uint_as_float(a.y << 16);
            v[j].w += __uint_as_float(a.y & 0xffff0000u);
            xr[idx] = v[j];
        }
        ss = fmaf(v[j].x, v[j].x, ss);
        ss = fmaf(v[j].y, v[j].y, ss);
        ss = fmaf(v[j].z, v[j].z, ss);
        ss = fmaf(v[j].w, v[j].w, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    uint2* o = (uint2*)(out + (size_t)i * dim);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = w4[idx];
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

extern "C" int gfa_add_rmsnorm(float* res, const void* y, const float* w, void* out, int n_rows,
                               int dim, float eps, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    const bf16_t* yp = (const bf16_t*)y;
    bf16_t* op = (bf16_t*)out;
    const bool vec = dim % 4 == 0 && dim <= 8192 && (uintptr_t)res % 16 == 0 &&
                     (uintptr_t)y % 8 == 0 && (uintptr_t)out % 8 == 0 && (uintptr_t)w % 16 == 0;
    if (!vec) add_rmsnorm_kernel<<<n_rows, 256, 0, stream>>>(res, yp, w, op, dim, eps);
    else if (dim <= 1024) add_rmsnorm_vec_kernel<1, 256><<<n_rows, 256, 0, stream>>>(res, yp, w, op, dim, eps);
    else if (dim <= 4096) add_rmsnorm_vec_kernel<1, 1024><<<n_rows, 1024, 0, stream>>>(res, yp, w, op, dim, eps);
    else add_rmsnorm_vec_kernel<2, 1024><<<n_rows, 1024, 0, stream>>>(res, yp, w, op, dim, eps);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// float32 matrix product: out[m, n] (+)= sum_k a[m, k] * w[n, k]
// 64x64 tile per workgroup of 256 threads, 4x4 outputs per thread, k in steps of 16 through
// shared memory.  Each output is one fused-multiply-add chain over k = 0..K-1 in order.
#define GF_BM 64
#define GF_BN 64
#define GF_BK 16
__global__ __launch_bounds__(256) void gemm_f32_kernel(
        const float* __restrict__ a, const float* __restrict__ w, float* __restrict__ out,
        int M, int N, int K, int lda, int ldo, int accumulate) {
    __shared__ float As[GF_BK][GF_BM + 4];
    __shared__ float Ws[GF_BK][GF_BN + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GF_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = threadIdx.x + i * 256;
            const int r = e >> 4, c = e & 15;
            const int k = k0 + c;
            const int m = m0 + r, n = n0 + r;
            As[c][r] = (m < M && k < K) ? a[(size_t)m * lda + k] : 0.f;
            Ws[c][r] = (n < N && k < K) ? w[(size_t)n * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GF_BK; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float* o = out + (size_t)m * ldo + n;
            *o = accumulate ? (*o + acc[i][j]) : acc[i][j];
        }
    }
}

extern "C" int gfa_gemm_f32(const float* a, const float* w, float* out, int M, int N, int K,
                            int lda, int ldo, int accumulate, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM);
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, w, out, M, N, K, lda, ldo, accumulate);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Rotary position encoding of q and k, and the write of k and v into the paged cache.
// qkv: [N, (H + 2*Hkv) * hd] rows of q heads, k heads, v heads (model.py:195-199).
// Pair i of a head is (2i, 2i+1) if layout == 0 (model.py:281-293) or (i, i + rot/2) if
// layout == 1; it is rotated by angle = float(position) * freqs[i], cos and sin in float.
// Elements beyond `rot` pass through.  q goes to q_out [N, H, hd]; k and v of token n go
// to page table[seq(n)][pos / PAGE], offset pos % PAGE (model.py:91-100, 206-207); keys as
// rows [offset, hd], values transposed [hd, offset] (see common.h).
template <typename T>
__global__ __launch_bounds__(256) void rope_cache_kernel(
        const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_pages,
        T* __restrict__ v_pages, const float* __restrict__ freqs, const int* __restrict__ tok_seq,
        const int* __restrict__ tok_pos, const int* __restrict__ table, int table_stride, int H,
        int Hkv, int hd, int rot, int layout) {
    // one thread per pair of elements: q and k heads first (rotated or passed through), then
    // the pairs of v; blockIdx.y walks the token's pairs in groups of 256
    const int n = blockIdx.x;
    const int half = hd / 2;
    const int rot_pairs = rot / 2;
    const int qk_slots = (H + Hkv) * half, v_slots = Hkv * half;
    const int pos = tok_pos[n];
    // cos and sin of this token's angles, once per workgroup
    extern __shared__ float cs[];                          // [rot_pairs][2]
    if (blockIdx.y * 256 < qk_slots) {
        for (int i = threadIdx.x; i < rot_pairs; i += 256)
            sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
        __syncthreads();
    }
    const int e = blockIdx.y * 256 + threadIdx.x;
    if (e >= qk_slots + v_slots) return;
    const T* row = qkv + (size_t)n * (H + 2 * Hkv) * hd;
    int page = 0;
    if (k_pages) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    if (e < qk_slots) {
        const int head = e / half, i = e - head * half;
        const T* src = row + (size_t)head * hd;
        if (head >= H && !k_pages) return;
        // where element d of this head goes: a row of q_out, or the key's place in its page
        T* const dst = head < H ? q_out + ((size_t)n * H + head) * hd
                                : k_pages + cache_region(page, head - H, Hkv, hd);
        auto place = [&](int d) { return head < H ? d : key_offset(off, d, hd); };
        if (i < rot_pairs) {
            const int ia = layout == 0 ? 2 * i : i;
            const int ib = layout == 0 ? 2 * i + 1 : i + rot_pairs;
            const float a = load_as_float(src + ia), b = load_as_float(src + ib);
            const float c = cs[2 * i], s = cs[2 * i + 1];
            store_from_float(dst + place(ia), a * c - b * s);
            store_from_float(dst + place(ib), b * c + a * s);
        } else {
            const int d0 = rot + 2 * (i - rot_pairs);      // elements rot .. hd-1 are copied
            dst[place(d0)] = src[d0];
            dst[place(d0 + 1)] = src[d0 + 1];
        }
    } else if (v_pages) {
        const int ev = e - qk_slots;
        const int g = ev / half, d = 2 * (ev - g * half);
        const T* vsrc = row + (size_t)(H + Hkv + g) * hd + d;
        v_pages[value_elem(page, g, d, off, Hkv, hd)] = vsrc[0];
        v_pages[value_elem(page, g, d + 1, off, Hkv, hd)] = vsrc[1];
    }
}

// The same for bfloat16 with interleaved pairs, eight elements (four pairs) per thread:
// 16-byte loads and stores for q and k.  Needs hd and rot to be multiples of 8.
__global__ __launch_bounds__(256) void rope_cache_bf16x8_kernel(
        const bf16_t* __restrict__ qkv, bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_pages,
        bf16_t* __restrict__ v_pages, const float* __restrict__ freqs,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, int H, int Hkv, int hd, int rot) {
    const int n = blockIdx.x;
    const int per_head = hd / 8;
    const int qk_chunks = (H + Hkv) * per_head, v_chunks = Hkv * per_head;
    const int pos = tok_pos[n];
    extern __shared__ float cs[];                          // [rot / 2][2]
    if (blockIdx.y * 256 < qk_chunks) {
        for (int i = threadIdx.x; i < rot / 2; i += 256)
            sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
        __syncthreads();
    }
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= qk_chunks + v_chunks) return;
    const int head = c / per_head, d0 = (c - head * per_head) * 8;
    union { uint4 u; bf16_t e[8]; } in, out;
    in.u = *(const uint4*)(qkv + ((size_t)n * (H + 2 * Hkv) + head) * hd + d0);
    int page = 0;
    if (k_pages && head >= H) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    if (head < H + Hkv) {
        if (d0 < rot) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float a = bf16_to_float(in.e[2 * p]), b = bf16_to_float(in.e[2 * p + 1]);
                const float c_ = cs[d0 + 2 * p], s_ = cs[d0 + 2 * p + 1];
                out.e[2 * p] = float_to_bf16(a * c_ - b * s_);
                out.e[2 * p + 1] = float_to_bf16(b * c_ + a * s_);
            }
        } else {
            out.u = in.u;
        }
        if (head < H) {
            *(uint4*)(q_out + ((size_t)n * H + head) * hd + d0) = out.u;
        } else if (k_pages) {
            *(uint4*)(k_pages + key_elem(page, head - H, off, d0, Hkv, hd)) = out.u;   // one chunk of 8 dims
        }
    } else if (v_pages) {
        const int g = head - H - Hkv;
#pragma unroll
        for (int j = 0; j < 8; ++j) v_pages[value_elem(page, g, d0 + j, off, Hkv, hd)] = in.e[j];
    }
}

// The same with the rows given as float partial sums of a sliced product, part [S, N, width]:
// the slices are added in order (the sum a kernel of its own would form), rotated and stored,
// so that the product's second kernel is this one.  The rotation then works on the float sums
// instead of their bfloat16 rounding.
__global__ __launch_bounds__(256) void rope_cache_sliced_bf16x8_kernel(
        const float* __restrict__ part, int S, size_t slice, bf16_t* __restrict__ q_out,
        bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const float* __restrict__ freqs,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, int H, int Hkv, int hd, int rot) {
    const int n = blockIdx.x;
    const int per_head = hd / 8;
    const int qk_chunks = (H + Hkv) * per_head, v_chunks = Hkv * per_head;
    const int pos = tok_pos[n];
    extern __shared__ float cs[];                          // [rot / 2][2]
    if (blockIdx.y * 256 < qk_chunks) {
        for (int i = threadIdx.x; i < rot / 2; i += 256)
            sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
        __syncthreads();
    }
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= qk_chunks + v_chunks) return;
    const int head = c / per_head, d0 = (c - head * per_head) * 8;
    const float* src = part + ((size_t)n * (H + 2 * Hkv) + head) * hd + d0;
    float v[8];
    {
        const float4 a = *(const float4*)src, b = *(const float4*)(src + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    for (int s = 1; s < S; ++s) {
        const float4 a = *(const float4*)(src + s * slice), b = *(const float4*)(src + s * slice + 4);
        v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
    }
    int page = 0;
    if (k_pages && head >= H) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    union { uint4 u; bf16_t e[8]; } out;
    if (head < H + Hkv) {
        if (d0 < rot) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float a = v[2 * p], b = v[2 * p + 1];
                const float c_ = cs[d0 + 2 * p], s_ = cs[d0 + 2 * p + 1];
                out.e[2 * p] = float_to_bf16(a * c_ - b * s_);
                out.e[2 * p + 1] = float_to_bf16(b * c_ + a * s_);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) out.e[j] = float_to_bf16(v[j]);
        }
        if (head < H) {
            *(uint4*)(q_out + ((size_t)n * H + head) * hd + d0) = out.u;
        } else if (k_pages) {
            *(uint4*)(k_pages + key_elem(page, head - H, off, d0, Hkv, hd)) = out.u;
        }
    } else if (v_pages) {
        const int g = head - H - Hkv;
#pragma unroll
        for (int j = 0; j < 8; ++j) v_pages[value_elem(page, g, d0 + j, off, Hkv, hd)] = float_to_bf16(v[j]);
    }
}

// part [S, n_tokens, (H + 2 Hkv) * hd] float; interleaved pairs, hd and rot multiples of 8.
extern "C" int gfa_rope_cache_write_sliced(const float* part, int S, void* q_out, void* k_pages,
                                           void* v_pages, const float* freqs, const int* tok_seq,
                                           const int* tok_pos, const int* table, int table_stride,
                                           int n_tokens, int H, int Hkv, int hd, int rot,
                                           hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (S <= 0 || hd % 8 != 0 || rot % 8 != 0 || rot > hd || (rot > 0 && !freqs))
        return (int)hipErrorInvalidValue;
    const dim3 grid(n_tokens, ((H + 2 * Hkv) * (hd / 8) + 255) / 256);
    const size_t slice = (size_t)n_tokens * (H + 2 * Hkv) * hd;
    rope_cache_sliced_bf16x8_kernel<<<grid, 256, (size_t)(rot > 0 ? rot : 2) * sizeof(float), stream>>>(
        part, S, slice, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, freqs, tok_seq, tok_pos,
        table, table_stride, H, Hkv, hd, rot);
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_rope_cache_write(const void* qkv, void* q_out, void* k_pages, void* v_pages,
                                    const float* freqs, const int* tok_seq, const int* tok_pos,
                                    const int* table, int table_stride, int n_tokens, int H,
                                    int Hkv, int hd, int rot, int layout, int is_bf16,
                                    hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (is_bf16 && layout == 0 && hd % 8 == 0 && rot % 8 == 0) {
        const dim3 grid8(n_tokens, ((H + 2 * Hkv) * (hd / 8) + 255) / 256);
        rope_cache_bf16x8_kernel<<<grid8, 256, (size_t)(rot > 0 ? rot : 2) * sizeof(float), stream>>>(
            (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, freqs, tok_seq,
            tok_pos, table, table_stride, H, Hkv, hd, rot);
        return GFA_LAUNCH_RESULT();
    }
    const dim3 grid(n_tokens, ((H + 2 * Hkv) * (hd / 2) + 255) / 256);
    if (is_bf16)
        rope_cache_kernel<bf16_t><<<grid, 256, (size_t)rot * sizeof(float), stream>>>(
            (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, freqs,
            tok_seq, tok_pos, table, table_stride, H, Hkv, hd, rot, layout);
    else
        rope_cache_kernel<float><<<grid, 256, (size_t)rot * sizeof(float), stream>>>(
            (const float*)qkv, (float*)q_out, (float*)k_pages, (float*)v_pages, freqs, tok_seq,
            tok_pos, table, table_stride, H, Hkv, hd, rot, layout);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Attention of each new token over its sequence's cache (model.py:209-211 with the mask of
// model.py:134,138): query head h reads kv head h / (H/Hkv); keys j with
// max(0, pos-window+1) <= j <= pos (window 0: from 0); scores scaled, softmax with running
// maximum, all in float.  One workgroup of 128 threads per (head, token); keys in chunks of
// 128, one key per thread for the scores, one output element per thread for the values.
#define AG_THREADS 128
#define AG_MAX_PER_THREAD 4            // head_dim <= 512
template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
        const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, T* __restrict__ out, int H, int Hkv,
        int hd, float scale, int window) {
    extern __shared__ float shared[];
    float* qs = shared;                 // [hd]
    float* sc = shared + hd;            // [AG_THREADS]
    float* scratch = sc + AG_THREADS;   // [16]
    const int n = blockIdx.x, h = blockIdx.y;     // tokens in x: a step may bring millions
    const int g = h / (H / Hkv);
    const int pos = tok_pos[n];
    const int* pages = table + (size_t)tok_seq[n] * table_stride;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const T* qrow = q + ((size_t)n * H + h) * hd;
    for (int d = threadIdx.x; d < hd; d += AG_THREADS) qs[d] = load_as_float(qrow + d);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[AG_MAX_PER_THREAD];
#pragma unroll
    for (int i = 0; i < AG_MAX_PER_THREAD; ++i) acc[i] = 0.f;

    for (int base = lo; base <= pos; base += AG_THREADS) {
        const int j = base + threadIdx.x;
        float s = -INFINITY;
        if (j <= pos) {
            const T* kr = k_pages + cache_region(pages[j / GFA_PAGE], g, Hkv, hd);
            float dot = 0.f;
            for (int d = 0; d < hd; ++d)
                dot = fmaf(qs[d], load_as_float(kr + key_offset(j % GFA_PAGE, d, hd)), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, block_max(s, scratch));
        const float alpha = expf(m - m_new);          // 0 on the first chunk (m = -inf)
        const float p = (j <= pos) ? expf(s - m_new) : 0.f;
        sc[threadIdx.x] = p;
        l = l * alpha + block_sum(p, scratch);        // contains the barrier that publishes sc
        const int count = (pos - base + 1 < AG_THREADS) ? pos - base + 1 : AG_THREADS;
#pragma unroll
        for (int i = 0; i < AG_MAX_PER_THREAD; ++i) {
            const int d = threadIdx.x + i * AG_THREADS;
            if (d < hd) {
                float a = acc[i] * alpha;
                for (int jj = 0; jj < count; ++jj) {
                    const int key = base + jj;
                    const T* vr = v_pages + value_elem(pages[key / GFA_PAGE], g, d,
                                                       key % GFA_PAGE, Hkv, hd);
                    a = fmaf(sc[jj], load_as_float(vr), a);
                }
                acc[i] = a;
            }
        }
        m = m_new;
        __syncthreads();
    }
    T* orow = out + ((size_t)n * H + h) * hd;
#pragma unroll
    for (int i = 0; i < AG_MAX_PER_THREAD; ++i) {
        const int d = threadIdx.x + i * AG_THREADS;
        if (d < hd) store_from_float(orow + d, acc[i] / l);
    }
}

extern "C" int gfa_attention_generic(const void* q, const void* k_pages, const void* v_pages,
                                     const int* tok_seq, const int* tok_pos, const int* table,
                                     int table_stride, void* out, int n_tokens, int H, int Hkv,
                                     int hd, float scale, int window, int is_bf16,
                                     hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (hd > AG_THREADS * AG_MAX_PER_THREAD || H > 65535) return (int)hipErrorInvalidValue;
    dim3 grid(n_tokens, H);
    const size_t shmem = (size_t)(hd + AG_THREADS + 16) * sizeof(float);
    if (is_bf16)
        attention_generic_kernel<bf16_t><<<grid, AG_THREADS, shmem, stream>>>(
            (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, tok_seq, tok_pos,
            table, table_stride, (bf16_t*)out, H, Hkv, hd, scale, window);
    else
        attention_generic_kernel<float><<<grid, AG_THREADS, shmem, stream>>>(
            (const float*)q, (const float*)k_pages, (const float*)v_pages, tok_seq, tok_pos,
            table, table_stride, (float*)out, H, Hkv, hd, scale, window);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// gate: out[n, i] = act(gu[n, i]) * gu[n, I + i], act = silu (model.py:227)
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I,
                                size_t total) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x) {
        const size_t n = e / I;
        const int i = (int)(e % I);
        const float a = load_as_float(gu + n * 2 * I + i);
        const float b = load_as_float(gu + n * 2 * I + I + i);
        store_from_float(out + e, (a / (1.f + expf(-a))) * b);
    }
}

// bfloat16 rows whose width is a multiple of 8: eight elements per thread, 16-byte accesses
__global__ __launch_bounds__(256) void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu,
                                                              bf16_t* __restrict__ out, int I8,
                                                              size_t total8) {
    const size_t e = blockIdx.x * (size_t)256 + threadIdx.x;
    if (e >= total8) return;
    const size_t n = e / I8;
    const int i = (int)(e - n * I8);
    const uint4 a = ((const uint4*)gu)[n * 2 * I8 + i], b = ((const uint4*)gu)[n * 2 * I8 + I8 + i];
    const bf16_t* ae = (const bf16_t*)&a;
    const bf16_t* be = (const bf16_t*)&b;
    uint4 o;
    bf16_t* oe = (bf16_t*)&o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float x = bf16_to_float(ae[j]);
        oe[j] = float_to_bf16((x / (1.f + expf(-x))) * bf16_to_float(be[j]));
    }
    ((uint4*)out)[e] = o;
}

extern "C" int gfa_silu_mul(const void* gu, void* out, int n_rows, int I, int is_bf16,
                            hipStream_t stream) {
    const size_t total = (size_t)n_rows * I;
    if (total == 0) return 0;
    if (is_bf16 && I % 8 == 0) {
        const size_t total8 = total / 8;
        silu_mul_bf16x8_kernel<<<(unsigned)((total8 + 255) / 256), 256, 0, stream>>>(
            (const bf16_t*)gu, (bf16_t*)out, I / 8, total8);
        return GFA_LAUNCH_RESULT();
    }
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (is_bf16)
        silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total);
    else
        silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, I, total);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// residual sum in float: res[e] += float(y[e])          (model.py:162-163)
template <typename T>
__global__ void add_into_kernel(float* __restrict__ res, const T* __restrict__ y, size_t total) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x)
        res[e] += load_as_float(y + e);
}

// bfloat16 addend, four elements per thread
__global__ __launch_bounds__(256) void add_into_bf16x4_kernel(float4* __restrict__ res,
                                                              const uint2* __restrict__ y,
                                                              size_t total4) {
    const size_t e = blockIdx.x * (size_t)256 + threadIdx.x;
    if (e >= total4) return;
    float4 r = res[e];
    const uint2 v = y[e];
    r.x += __uint_as_float(v.x << 16);
    r.y += __uint_as_float(v.x & 0xffff0000u);
    r.z += __uint_as_float(v.y << 16);
    r.w += __uint_as_float(v.y & 0xffff0000u);
    res[e] = r;
}

extern "C" int gfa_add_into(float* res, const void* y, size_t total, int y_bf16,
                            hipStream_t stream) {
    if (total == 0) return 0;
    if (y_bf16 && total % 4 == 0 && ((uintptr_t)res % 16 == 0) && ((uintptr_t)y % 8 == 0)) {
        const size_t total4 = total / 4;
        add_into_bf16x4_kernel<<<(unsigned)((total4 + 255) / 256), 256, 0, stream>>>(
            (float4*)res, (const uint2*)y, total4);
        return GFA_LAUNCH_RESULT();
    }
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (y_bf16)
        add_into_kernel<bf16_t><<<blocks, 256, 0, stream>>>(res, (const bf16_t*)y, total);
    else
        add_into_kernel<float><<<blocks, 256, 0, stream>>>(res, (const float*)y, total);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// x[e] = scale * x[e], then, if cap > 0, cap * tanh(x[e] / cap): a factor on the embedded
// rows or on the logits, and a soft cap of the logits, for plans that state one.
__global__ void scale_cap_kernel(float* __restrict__ x, size_t total, float scale, float cap) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x) {
        float v = x[e] * scale;
        if (cap > 0.f) v = cap * tanhf(v / cap);
        x[e] = v;
    }
}

extern "C" int gfa_scale_cap(float* x, size_t total, float scale, float cap, hipStream_t stream) {
    if (total == 0) return 0;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    scale_cap_kernel<<<blocks, 256, 0, stream>>>(x, total, scale, cap);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// naive matrix product with bfloat16 operands and float accumulation, one thread per
// output: the plain counterpart of the fast bfloat16 kernels (tests only).
__global__ void gemm_bf16_naive_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                       float* __restrict__ out, int M, int N, int K) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x, m = blockIdx.y;
    if (n >= N || m >= M) return;
    float acc = 0.f;
    for (int k = 0; k < K; ++k)
        acc = fmaf(bf16_to_float(a[(size_t)m * K + k]), bf16_to_float(w[(size_t)n * K + k]), acc);
    out[(size_t)m * N + n] = acc;
}

extern "C" int gfa_gemm_bf16_naive(const void* a, const void* w, float* out, int M, int N, int K,
                                   hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 65535) return (int)hipErrorInvalidValue;     // rows ride in the grid's second dimension
    dim3 grid((N + 255) / 256, M);
    gemm_bf16_naive_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, out, M, N, K);
    return GFA_LAUNCH_RESULT();
}
