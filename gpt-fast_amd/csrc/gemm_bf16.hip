// Few-row matrix products with bfloat16 operands for decoding: out = x W^T with
// x [M, K] (M <= 64) and W [N, K], both row-major bfloat16, float accumulation.
//
// With few rows the product is bound by reading W once from HBM, so the kernels are
// organised around that stream: every wavefront owns a few rows of W and reads them
// front to back in 16-byte pieces per lane (1 KiB contiguous per wave and load), keeps
// one float accumulator per (row of W, row of x) and reduces over the lanes at the end.
// x is small and stays in cache: W is read with non-temporal loads so that the stream does
// not displace it, for every workgroup reads all of x again.  One row uses v_dot2_f32_bf16
// (two multiply-adds per lane and instruction, float accumulate); more rows the matrix cores
// (second kernel below).
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
__device__ __forceinline__ void skinny_store(void* out, int ldo, int m, int n, float v, float gate_v,
                                             int out_pad = 0) {
    if (MODE == 4) return;                     // the rotary epilogue stores by itself
    if (MODE == 3 && out_pad) {
        ((bf16_t*)out)[chunked_elem(m, n, out_pad)] = float_to_bf16(silu(v) * gate_v);
        return;
    }
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
                    wa[r].u = stream_load16(wrow[r] + k0 + c * 8);
                    wb[r].u = stream_load16(wrow[r] + k0 + (c + 64) * 8);
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
                for (int r = 0; r < WR; ++r) wa[r].u = stream_load16(wrow[r] + k0 + c * 8);
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
#define GFA_MAX_SHARE_COPIES 64

union Frag8 {
    uint4 u;
    bf16x8_t v;
};

// What the fused variants need beside the product itself.
struct SkinnyExtra {
    float eps;                // of the norm whose row factor this product applies (below)
    // MODE 4: the columns are q heads, k heads, v heads (model.py:195-199); q and k pairs
    // (2i, 2i+1) are rotated by tok_pos * freqs[i] (model.py:281-293), q goes to q_out
    // [M, H, hd], k and v into the pages (model.py:91-100) unless k_pages is null
    bf16_t* q_out;
    bf16_t* k_pages;
    bf16_t* v_pages;
    const float* freqs;
    const int* tok_seq;
    const int* tok_pos;
    const int* table;
    int table_stride, H, Hkv, hd, rot;
    // A norm spread over two kernels (one tile of rows).  The kernel that completes the
    // residual stream (MODE 2) also writes xg_out = bfloat16(new residual * next_g) (chunked) and
    // ssq_out [gfa_skinny_workgroups(2, M, N), share_rows]: each workgroup's share of its rows' sums of squares (float,
    // from the float residual).  The next product takes xg as its x, adds the shares in a fixed
    // order (ssq_in [t_in, share_rows]) and scales its result by rsqrt(sum / K + eps): a factor per row
    // commutes with the product, so this is the RMS norm of model.py:236-241.
    bf16_t* xg_out;
    const float* next_g;
    float* ssq_out;
    const float* ssq_in;
    int t_in;
    int share_off;            // byte offset in LDS of the waves' pieces for the shares
    int share_copies;         // copy instructions per wave that bring the shares into LDS
    int share_rows;           // rows per share record: 4, 8, 16, 32 or 64 (the least that holds M)
    // chunked rows (see chunked_elem): x is read so if x_pad > 0; the gate's output (MODE 3)
    // is written so if out_pad > 0; xg_out always is, with share_rows as its pad
    int x_pad, out_pad;
};

// Rows per record of the sums-of-squares shares for M rows of x.
extern "C" int gfa_share_rows(int M) { return M <= 4 ? 4 : M <= 8 ? 8 : M <= 16 ? 16 : M <= 32 ? 32 : 64; }

// TILES = 2 (nine to 48 rows of x, wide matrices, not the gate): a workgroup takes two
// tiles of W's rows, one below the other, against the same fragments of x.  With sixteen
// rows every workgroup reads as many bytes of x as of W; two tiles halve that, at half as
// many workgroups, which pays where those still fill the chip.
// XPL = 2 or 4 (several tiles of x rows, CT > 1): the last tile holds at most eight or four
// rows, and its idle operand columns carry later steps of k as with XP: with 17 to 24 rows
// the second tile then takes two load instructions per piece instead of four (a load
// instruction costs the same whether all its lanes are rows or one is).
template <int CT, int MODE, int XP = 1, bool XF = false, int TILES = 1, int XPL = 1>
__global__ __launch_bounds__(512) void skinny_mfma_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M,
        int N, int K, int ldo, int gate_rows, int th, SkinnyExtra ex) {
    static_assert(TILES == 1 || (TILES == 2 && CT <= 3 && MODE != 3), "two tiles: up to 48 rows of x, no gate");
    constexpr int RT = (MODE == 3) ? 2 : TILES;          // tiles of W's rows multiplied per x fragment
    constexpr int NT = (MODE == 3) ? 1 : TILES;          // tiles of output columns per workgroup
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, NW = blockDim.x >> 6;
    // th (12..16) rows of W per tile: the host picks it so that the tiles divide evenly
    // over the compute units; operand rows th..15 repeat row th - 1 and are never stored
    const int n0 = blockIdx.x * th * NT;
    char* stage = smem + (size_t)wave * (RT * SM_TILE);
    const int lrow = lane >> 4, lchunk = lane & 15;      // loading: row lrow + 4 j, 16-byte chunk
    const int fi = lane & 15, fg = lane >> 4;            // multiplying: row / column fi, k group fg
    const int T = (K + SM_SUBK - 1) / SM_SUBK;
    const int t_begin = (int)((long)wave * T / NW), t_end = (int)((long)(wave + 1) * T / NW);

    floatx4_t acc[RT][CT];
    float ssq[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        ssq[ct] = 0.f;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][ct] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    const bf16_t* wsrc[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = lrow + 4 * j;
            int n = n0 + (MODE == 3 ? 0 : rt * th) + (r < th ? r : th - 1);
            if (n >= N) n = N - 1;                       // clamped rows are computed, not stored
            wsrc[rt][j] = w + (size_t)(n + (MODE == 3 ? rt * gate_rows : 0)) * K + lchunk * 8;
        }
    // two register sets: while piece t is multiplied, pieces t + 1 and t + 2 are in flight
    uint4 regs_a[RT][4], regs_b[RT][4];
    auto load_piece = [&](int t, uint4 (&regs)[RT][4]) {
        const int k = t * SM_SUBK + lchunk * 8;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                regs[rt][j] = (k < K) ? stream_load16(wsrc[rt][j] + t * SM_SUBK) : make_uint4(0, 0, 0, 0);
    };
    auto stage_piece = [&](uint4 (&regs)[RT][4]) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *(uint4*)(stage + rt * SM_TILE + (lrow + 4 * j) * SM_PITCH + lchunk * 16) = regs[rt][j];
    };
    // The x fragments of a piece are requested a whole piece ahead, and before the prefetch of
    // the W piece issued next: loads return in order, so when a piece is multiplied its x has
    // long been asked for and waiting for it lets two later pieces of W stay in flight.
    //
    // XP = 2 or 4 (at most eight or four rows of x, CT == 1): the other columns of the x
    // operand stand for no row, and what a matrix instruction makes of them is never stored.
    // So the sixteen lanes of a group are 16 / XP rows times XP steps of 32 k: part q of the
    // lanes loads, in the same instruction, the chunk that part 0 needs q steps later - the
    // next pieces of the rows' 128-byte lines - and a rotation of the group by q * 16 / XP
    // lanes brings it down when that step is multiplied: 1 / XP of the load instructions
    // for x, each using whole lines.
    constexpr int XS = SM_SUBK / 32;
    constexpr int XL = XS / XP;                          // loads of x per piece and tile of rows
    constexpr int XROWS = 16 / XP;
    static_assert(XP == 1 || CT == 1, "shared operand columns need a single tile of rows");
    static_assert(XPL == 1 || (CT > 1 && XP == 1 && !XF), "a narrower last tile needs several tiles");
    constexpr int XLL = XS / XPL, XROWSL = 16 / XPL;     // of the last tile of rows
    uint4 x_a[XL][CT], x_b[XL][CT];
    auto load_x = [&](int t, uint4 (&xraw)[XL][CT]) {
#pragma unroll
        for (int s = 0; s < XL; ++s) {
            // XF: load s of a pair takes rows 8 (s & 1) .. + 7, its lanes 8..15 the later step
            const int kk = XF ? t * SM_SUBK + (((s & ~1) + (fi >> 3)) * 4 + fg) * 8
                              : t * SM_SUBK + ((XP * s + fi / XROWS) * 4 + fg) * 8;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                if (XPL > 1 && ct == CT - 1) {           // the narrower last tile: fewer loads
                    if (s < XLL) {
                        const int kl = t * SM_SUBK + ((XPL * s + fi / XROWSL) * 4 + fg) * 8;
                        const int m = ct * 16 + fi % XROWSL;
                        const bf16_t* src = ex.x_pad ? x + chunked_elem(m, kl, ex.x_pad) : x + (size_t)m * K + kl;
                        xraw[s][ct] = (m < M && kl < K) ? *(const uint4*)src : make_uint4(0, 0, 0, 0);
                    }
                    continue;
                }
                const int m = XF ? ct * 16 + 8 * (s & 1) + (fi & 7) : ct * 16 + fi % XROWS;
                const bf16_t* src = ex.x_pad ? x + chunked_elem(m, kk, ex.x_pad) : x + (size_t)m * K + kk;
                xraw[s][ct] = (m < M && kk < K) ? *(const uint4*)src : make_uint4(0, 0, 0, 0);
            }
        }
    };
    // XF (nine to sixteen rows, XP == 1): every column of the operand is a row, but a load can
    // still use whole lines: of a pair of steps, the first load takes rows 0..7 and the second
    // rows 8..15, in each the lanes 8..15 the later step; halves are exchanged by the same
    // rotation when a step is multiplied.
    // lanes i of every group of sixteen get the value of lane (i + N) mod 16
    #define GFA_ROTATE_DOWN(v, N) __builtin_amdgcn_update_dpp(0, (int)(v), 0x120 + ((16 - (N)) & 15), 0xf, 0xf, false)
    auto multiply_piece = [&](int t, const uint4 (&xraw)[XL][CT]) {
#pragma unroll
        for (int s = 0; s < XS; ++s) {
            Frag8 b[CT];
            if (XF) {
                // rows 0..7 of step s sit in the pair's first load (lanes 0..7 if s is even,
                // 8..15 if odd), rows 8..15 in its second: own lanes or the other half's
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const uint4 lo = xraw[s & ~1][ct], hi = xraw[s | 1][ct];
                    const uint4 moved = (s & 1) ? lo : hi;     // the one that has to change halves
                    uint4 r;
                    r.x = GFA_ROTATE_DOWN(moved.x, 8); r.y = GFA_ROTATE_DOWN(moved.y, 8);
                    r.z = GFA_ROTATE_DOWN(moved.z, 8); r.w = GFA_ROTATE_DOWN(moved.w, 8);
                    const bool low = fi < 8;
                    const uint4 a0 = (s & 1) ? r : lo, a1 = (s & 1) ? hi : r;
                    b[ct].u = make_uint4(low ? a0.x : a1.x, low ? a0.y : a1.y, low ? a0.z : a1.z, low ? a0.w : a1.w);
                }
            } else {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) b[ct].u = xraw[s / XP][ct];
            }
            if (XPL > 1) {                               // the last tile: its load of this group of steps,
                uint4 v = xraw[s / XPL][CT - 1];         // rotated down to the step's lanes
                const int q = s % XPL;
                if (q * XROWSL == 4) {
                    v.x = GFA_ROTATE_DOWN(v.x, 4); v.y = GFA_ROTATE_DOWN(v.y, 4);
                    v.z = GFA_ROTATE_DOWN(v.z, 4); v.w = GFA_ROTATE_DOWN(v.w, 4);
                } else if (q * XROWSL == 8) {
                    v.x = GFA_ROTATE_DOWN(v.x, 8); v.y = GFA_ROTATE_DOWN(v.y, 8);
                    v.z = GFA_ROTATE_DOWN(v.z, 8); v.w = GFA_ROTATE_DOWN(v.w, 8);
                } else if (q * XROWSL == 12) {
                    v.x = GFA_ROTATE_DOWN(v.x, 12); v.y = GFA_ROTATE_DOWN(v.y, 12);
                    v.z = GFA_ROTATE_DOWN(v.z, 12); v.w = GFA_ROTATE_DOWN(v.w, 12);
                }
                b[CT - 1].u = v;
            }
            if (XP > 1 && s % XP != 0) {
                const int q = s % XP;
                if (q * XROWS == 4) {
                    b[0].u.x = GFA_ROTATE_DOWN(b[0].u.x, 4); b[0].u.y = GFA_ROTATE_DOWN(b[0].u.y, 4);
                    b[0].u.z = GFA_ROTATE_DOWN(b[0].u.z, 4); b[0].u.w = GFA_ROTATE_DOWN(b[0].u.w, 4);
                } else if (q * XROWS == 8) {
                    b[0].u.x = GFA_ROTATE_DOWN(b[0].u.x, 8); b[0].u.y = GFA_ROTATE_DOWN(b[0].u.y, 8);
                    b[0].u.z = GFA_ROTATE_DOWN(b[0].u.z, 8); b[0].u.w = GFA_ROTATE_DOWN(b[0].u.w, 8);
                } else {
                    b[0].u.x = GFA_ROTATE_DOWN(b[0].u.x, 12); b[0].u.y = GFA_ROTATE_DOWN(b[0].u.y, 12);
                    b[0].u.z = GFA_ROTATE_DOWN(b[0].u.z, 12); b[0].u.w = GFA_ROTATE_DOWN(b[0].u.w, 12);
                }
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
    };
    #undef GFA_ROTATE_DOWN
    if (t_begin < t_end) {
        load_piece(t_begin, regs_a);
        load_x(t_begin, x_a);
    }
    if (t_begin + 1 < t_end) load_piece(t_begin + 1, regs_b);
    // What the epilogue of wave 0 reads is requested now, behind the first pieces of W, so
    // that its latency (and the rotation's sine and cosine) passes while W streams.
    float4 res_pre[NT][CT], g_pre[NT][CT];               // MODE 2: the residual's old values, next norm's weights
    bool res_ok[NT][CT];
    float rot_cs[NT][CT][2], rot_sn[NT][CT][2];          // MODE 4: cosine and sine of this lane's two pairs
    int rot_pos[CT], rot_page[CT];                       // a token's page serves all tiles of columns
    constexpr bool ROT_EARLY = MODE == 4;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) rot_pos[ct] = rot_page[ct] = 0;
#pragma unroll
    for (int ot = 0; ot < NT; ++ot) {
        const int nb = n0 + ot * th;                     // first column of this output tile
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            rot_cs[ot][ct][0] = rot_cs[ot][ct][1] = 1.f;
            rot_sn[ot][ct][0] = rot_sn[ot][ct][1] = 0.f;
            res_ok[ot][ct] = false;
            if (MODE == 2 && wave == 0) {
                const int m = ct * 16 + fi, n = nb + fg * 4;
                res_ok[ot][ct] = m < M && n + 3 < N && (ldo & 3) == 0 && fg * 4 + 3 < th;
                if (res_ok[ot][ct]) {
                    res_pre[ot][ct] = *(const float4*)((const float*)out + (size_t)m * ldo + n);
                    if (ex.xg_out) g_pre[ot][ct] = *(const float4*)(ex.next_g + n);
                }
            }
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const int m = ct * 16 + fi;
            if (ROT_EARLY && wave == 0 && m < M && nb + fg * 4 < N && fg * 4 < th) {
                const int n = nb + fg * 4;
                const int head = n / ex.hd, d = n - head * ex.hd;
                rot_pos[ct] = ex.tok_pos[m];
                if (head >= ex.H && ex.k_pages)
                    rot_page[ct] = ex.table[(size_t)ex.tok_seq[m] * ex.table_stride + rot_pos[ct] / GFA_PAGE];
                if (head < ex.H + ex.Hkv) {
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr)
                        if (d + 2 * pr < ex.rot)
                            sincosf((float)rot_pos[ct] * ex.freqs[(d + 2 * pr) >> 1], &rot_sn[ot][ct][pr],
                                    &rot_cs[ot][ct][pr]);
                }
            }
        }
    }
    // second half of a two-kernel norm.  A share record holds R = share_rows rows side by
    // side; one copy instruction of a wave takes 64 / R records (lane l: row l % R of record
    // l / R), wave w takes the record groups w, w + NW, ...  The copies go straight into a
    // wave-private piece of LDS - no register waits for them, so nothing below is held up -
    // and are added after the product.  Every workgroup reads all shares, so their bytes
    // count: hence the narrow records for few rows.
    // copy instructions per wave: as many as bring in all records (the launcher sizes the LDS
    // piece by it), at most GFA_MAX_SHARE_COPIES; records beyond are read at the end, one
    // round trip after the other
    const int SHARES = ex.share_copies;
    const bool chained = ex.ssq_in != nullptr;
    float* share_lds = (float*)(smem + ex.share_off) + wave * (SHARES * 64);
    const int R = ex.share_rows, per_copy = R ? 64 / R : 4;
    if (chained) {
        for (int j = 0; j < SHARES; ++j) {
            const int first = per_copy * (wave + NW * j);
            if (first < ex.t_in) {                         // wave-uniform
                const int rec = first + lane / R;
                const float* src = ex.ssq_in + (size_t)(rec < ex.t_in ? rec : 0) * R + lane % R;
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)src,
                    (__attribute__((address_space(3))) void*)(share_lds + j * 64), 4, 0, 0);
            }
        }
    }
    for (int t = t_begin; t < t_end; t += 2) {
        if (t + 1 < t_end) load_x(t + 1, x_b);
        stage_piece(regs_a);
        if (t + 2 < t_end) load_piece(t + 2, regs_a);
        multiply_piece(t, x_a);
        if (t + 1 < t_end) {
            if (t + 2 < t_end) load_x(t + 2, x_a);
            stage_piece(regs_b);
            if (t + 3 < t_end) load_piece(t + 3, regs_b);
            multiply_piece(t + 1, x_b);
        }
    }
    if (chained) {                                       // fixed order: lane, lanes of a row, waves
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the copies into LDS have landed
        float pre_ssq = 0.f;
        for (int j = 0; j < SHARES; ++j) {
            const int rec = per_copy * (wave + NW * j) + lane / R;
            if (rec < ex.t_in) pre_ssq += share_lds[j * 64 + lane];
        }
        for (int rec = per_copy * (wave + NW * SHARES) + lane / R; rec < ex.t_in; rec += per_copy * NW)
            pre_ssq += ex.ssq_in[(size_t)rec * R + lane % R];
        // lanes l, l + R, l + 2 R, ... hold parts of row l % R: a butterfly in a fixed order
        for (int step = R; step < 64; step <<= 1) {
            const float other = __shfl_xor(pre_ssq, step, GFA_WAVE);
            pre_ssq = (lane & step) ? other + pre_ssq : pre_ssq + other;
        }
        // now every lane l holds the wave's part of the sum of row l % R; row 16 ct + fi is this
        // lane's in tile ct
        if (CT == 1) {
            ssq[0] = pre_ssq;                            // R <= 16: row fi is lane fi's, whatever fg
        } else {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) ssq[ct] = __shfl(pre_ssq, ct * 16 + fi, GFA_WAVE);
        }
    }
    if (NW > 1) {
        __syncthreads();                                 // staging is done; reuse it for the sums
        floatx4_t* red = (floatx4_t*)smem;
        float* red_s = (float*)(smem + (size_t)NW * RT * CT * 64 * sizeof(floatx4_t));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) red[((wave * RT + rt) * CT + ct) * 64 + lane] = acc[rt][ct];
        if (chained && fg == 0) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) red_s[(wave * CT + ct) * 16 + fi] = ssq[ct];
        }
        __syncthreads();
        if (wave != 0) return;
        for (int wv = 1; wv < NW; ++wv) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc[rt][ct] += red[((wv * RT + rt) * CT + ct) * 64 + lane];
            if (chained) {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) ssq[ct] += red_s[(wv * CT + ct) * 16 + fi];
            }
        }
    }
    float part_ssq[CT];                                  // MODE 2 with xg_out: this lane's r^2 per tile of rows
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) part_ssq[ct] = 0.f;
    if (chained) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const float rs = rsqrtf(ssq[ct] / (float)K + ex.eps);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) acc[rt][ct] *= rs;
        }
    }
#pragma unroll
    for (int ot = 0; ot < NT; ++ot)                      // the workgroup's tiles of output columns
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = ct * 16 + fi;
        const int nb = n0 + ot * th;                     // first column of this tile
        if (m >= M) continue;
        if (MODE == 4) {
            // columns nb + 4 fg .. +3 of token m: two rotary pairs of one head
            const int n = nb + fg * 4;
            if (n >= N || fg * 4 >= th) continue;        // th is a multiple of 4 here
            const int hd = ex.hd, head = n / hd, d = n - head * hd;
            const int pos = rot_pos[ct];
            float v[4] = {acc[ot][ct][0], acc[ot][ct][1], acc[ot][ct][2], acc[ot][ct][3]};
            if (head < ex.H + ex.Hkv) {
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const int dd = d + 2 * pr;
                    if (dd < ex.rot) {
                        const float sn = rot_sn[ot][ct][pr], cs = rot_cs[ot][ct][pr];
                        const float a = v[2 * pr], bb = v[2 * pr + 1];
                        v[2 * pr] = a * cs - bb * sn;
                        v[2 * pr + 1] = bb * cs + a * sn;
                    }
                }
            }
            Frag8 pk;
            bf16_t* e = (bf16_t*)&pk.u;
#pragma unroll
            for (int j = 0; j < 4; ++j) e[j] = float_to_bf16(v[j]);
            if (head < ex.H) {
                *(uint2*)(ex.q_out + ((size_t)m * ex.H + head) * hd + d) = make_uint2(pk.u.x, pk.u.y);
            } else if (ex.k_pages) {
                const int page = rot_page[ct];
                const int off = pos % GFA_PAGE;
                if (head < ex.H + ex.Hkv) {
                    *(uint2*)(ex.k_pages + key_elem(page, head - ex.H, off, d, ex.Hkv, hd)) =
                        make_uint2(pk.u.x, pk.u.y);
                } else {
                    const int g = head - ex.H - ex.Hkv;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        ex.v_pages[value_elem(page, g, d + j, off, ex.Hkv, hd)] = e[j];
                }
            }
        } else if (MODE == 2 && res_ok[ot][ct]) {
            float4 r = res_pre[ot][ct];                  // the same sums as skinny_store<2>
            r.x += acc[ot][ct][0];
            r.y += acc[ot][ct][1];
            r.z += acc[ot][ct][2];
            r.w += acc[ot][ct][3];
            *(float4*)((float*)out + (size_t)m * ldo + nb + fg * 4) = r;
            if (ex.xg_out) {                             // first half of the next norm; N == ldo
                const float4 g = g_pre[ot][ct];
                Frag8 pk;
                bf16_t* e = (bf16_t*)&pk.u;
                e[0] = float_to_bf16(r.x * g.x);
                e[1] = float_to_bf16(r.y * g.y);
                e[2] = float_to_bf16(r.z * g.z);
                e[3] = float_to_bf16(r.w * g.w);
                *(uint2*)(ex.xg_out + chunked_elem(m, nb + fg * 4, ex.share_rows)) = make_uint2(pk.u.x, pk.u.y);
                part_ssq[ct] += fmaf(r.x, r.x, fmaf(r.y, r.y, fmaf(r.z, r.z, r.w * r.w)));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = nb + fg * 4 + j;
                if (n < N && fg * 4 + j < th)
                    skinny_store<MODE>(out, ldo, m, n, acc[ot][ct][j], MODE == 3 ? acc[RT - 1][ct][j] : 0.f, ex.out_pad);
            }
        }
    }
    if (MODE == 2 && ex.xg_out) {                        // this workgroup's share, rows side by side
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float p = part_ssq[ct];
            p += __shfl_xor(p, 16, GFA_WAVE);
            p += __shfl_xor(p, 32, GFA_WAVE);
            if (fg == 0 && ct * 16 + fi < ex.share_rows)
                ex.ssq_out[(size_t)blockIdx.x * ex.share_rows + ct * 16 + fi] = p;
        }
        // a record is wider than the tiles of rows with 33..48 rows: the rest is zero
        if (fg == 1 && CT * 16 + fi < ex.share_rows)
            ex.ssq_out[(size_t)blockIdx.x * ex.share_rows + CT * 16 + fi] = 0.f;
    }
}

// Compute units of the current device (asked once).
static int compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        hipGetDevice(&dev);
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        cus = n > 0 ? n : 1;
    }
    return cus;
}

// Rows of W per workgroup (12..16, in steps of `step`) for a product with N output columns:
// the height at which the compute unit with the most tiles streams the fewest rows - with
// 16 rows, 6144 columns are 384 tiles on 256 compute units, half of which stream twice as
// much as the others; with 12 rows they are 512, two each.  The taller tile on a tie.  Not
// below 12: every tile reads all of x, so lower tiles cost in x what they save in W (10240
// columns at 8 rows, 1280 tiles for 640, measured 54 against 41 us at 16 rows of x).
static int pick_tile_rows(int N, int step, int nt = 1) {
    const int cus = compute_units();
    const long tiles16 = (N + 16 * nt - 1) / (16 * nt);
    const long cost16 = ((tiles16 + cus - 1) / cus) * 16;
    int best = 16;
    long best_cost = cost16;
    for (int th = 16 - step; th >= 12; th -= step) {
        const long tiles = (N + th * nt - 1) / (th * nt);
        const long cost = ((tiles + cus - 1) / cus) * th;
        if (cost < best_cost) {
            best = th;
            best_cost = cost;
        }
    }
    // a lower tile costs a little by itself (more workgroups, shorter runs of rows per load):
    // it has to save a twentieth of the rows the busiest compute unit streams
    return best_cost * 20 <= cost16 * 19 ? best : 16;
}

// Tiles of W's rows per workgroup: two for nine to 48 rows of x where the workgroups
// still fill three quarters of the chip (measured on 256 compute units at sixteen rows of x:
// 8192 x 28672 89 -> 79 us, 8192 x 8192 30.6 -> 26.5, 6144 x 4096 14.2 -> 12.8; with 4096 rows
// of W, 128 workgroups, a loss of a fifth).  Not the gate, which multiplies two sets of rows
// against the same x already: with two tiles of each, 242 registers, the step at sixteen rows
// lost 5 % (8B and 70B shapes) although the kernel alone gained 3 %.
static int tiles_per_workgroup(int mode, int M, int N) {
    // 33..48 rows: only where the registers hold it (the plain epilogues)
    const int most = (mode == 2 || mode == 4) ? 32 : 48;
    return (mode != 3 && M > 8 && M <= most && N >= 24 * compute_units()) ? 2 : 1;
}

// Tile height the launcher below uses for this mode, these rows of x and this width.
static int tile_rows(int mode, int M, int N) {
    return pick_tile_rows(N, (mode == 2 || mode == 4) ? 4 : 1, tiles_per_workgroup(mode, M, N));
}

// Workgroups the launcher below starts for this mode, M <= 16 rows of x and N columns (the
// two-kernel norm's shares are one record per workgroup of mode 2, so its callers size
// their buffers by it).
extern "C" int gfa_skinny_workgroups(int mode, int M, int N) {
    const int per = (M <= 16 ? tile_rows(mode, M, N) : 16) * tiles_per_workgroup(mode, M, N);
    return (N + per - 1) / per;
}

template <int MODE>
static int launch_skinny_mfma(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K,
                              int ldo, int gate_rows, const SkinnyExtra& ex, hipStream_t stream) {
    const int ct = (M + 15) / 16;
    // the epilogues that add into the residual stream or rotate pairs work on groups of
    // four columns: their tiles are 12 or 16 rows high
    const int nt = tiles_per_workgroup(MODE, M, N);
    const int th = ct == 1 ? tile_rows(MODE, M, N) : 16;
    const int tiles = (N + th * nt - 1) / (th * nt);     // workgroups
    const int RT = (MODE == 3) ? 2 : nt;                 // tiles of W staged per wave
    const int pieces = (K + SM_SUBK - 1) / SM_SUBK;
    int nw = 1;                                          // waves per tile: aim at >= 2048 waves,
    const int nw_max = (MODE == 3) ? 4 : 8;
    // at least four waves per tile where K allows: one wave walking sixteen rows alone
    // streams measurably slower than four that share them
    while (nw < nw_max && (tiles * nw < 2048 || nw < 4) && pieces >= 4 * nw) nw *= 2;
    size_t shmem = (size_t)nw * RT * SM_TILE;
    const size_t red = (size_t)nw * RT * ct * 64 * sizeof(floatx4_t) + (size_t)nw * ct * 16 * sizeof(float);
    if (nw > 1 && red > shmem) shmem = red;
    while (shmem > 96 * 1024 && nw > 1) {                // keep two workgroups per compute unit
        nw /= 2;
        shmem = (size_t)nw * RT * SM_TILE;
        const size_t r2 = (size_t)nw * RT * ct * 64 * sizeof(floatx4_t) + (size_t)nw * ct * 16 * sizeof(float);
        if (nw > 1 && r2 > shmem) shmem = r2;
    }
    SkinnyExtra exl = ex;
    if (ex.ssq_in) {                                     // the waves' pieces for the norm's shares
        const int per_copy = 64 / ex.share_rows;         // records per copy instruction
        int copies = (ex.t_in + per_copy * nw - 1) / (per_copy * nw);
        if (copies > GFA_MAX_SHARE_COPIES) copies = GFA_MAX_SHARE_COPIES;
        while (copies > 1 && shmem + (size_t)nw * copies * 64 * sizeof(float) > 128 * 1024) --copies;
        exl.share_off = (int)shmem;
        exl.share_copies = copies;
        shmem += (size_t)nw * copies * 64 * sizeof(float);
    }
#define GFA_LAUNCH_MFMA_L(CTV, XPV, XFV, NTV, XPLV)                                                    \
    do {                                                                                          \
        static bool raised = false;                                                               \
        if (!raised) {                                                                            \
            hipFuncSetAttribute((const void*)skinny_mfma_kernel<CTV, MODE, XPV, XFV, NTV, XPLV>,       \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);          \
            raised = true;                                                                        \
        }                                                                                         \
        skinny_mfma_kernel<CTV, MODE, XPV, XFV, NTV, XPLV><<<tiles, nw * 64, shmem, stream>>>(x, w, out, M, N, K, ldo, gate_rows, th, exl); \
    } while (0)
#define GFA_LAUNCH_MFMA(CTV, XPV, XFV, NTV) GFA_LAUNCH_MFMA_L(CTV, XPV, XFV, NTV, 1)
    switch (ct) {
        case 1:                                          // columns of the x operand that stand
            if (M <= 4) GFA_LAUNCH_MFMA(1, 4, false, 1);   // for no row carry later steps of k
            else if (M <= 8) GFA_LAUNCH_MFMA(1, 2, false, 1);
            else if (nt == 2) GFA_LAUNCH_MFMA(1, 1, true, (MODE == 3 ? 1 : 2));
            else GFA_LAUNCH_MFMA(1, 1, true, 1);
            break;
        case 2:                                          // 17..20, ..24 rows: a narrower second tile
            if (M <= 20) {
                if (nt == 2) GFA_LAUNCH_MFMA_L(2, 1, false, (MODE == 3 ? 1 : 2), 4);
                else GFA_LAUNCH_MFMA_L(2, 1, false, 1, 4);
            } else if (M <= 24) {
                if (nt == 2) GFA_LAUNCH_MFMA_L(2, 1, false, (MODE == 3 ? 1 : 2), 2);
                else GFA_LAUNCH_MFMA_L(2, 1, false, 1, 2);
            } else {
                if (nt == 2) GFA_LAUNCH_MFMA(2, 1, false, (MODE == 3 ? 1 : 2));
                else GFA_LAUNCH_MFMA(2, 1, false, 1);
            }
            break;
        case 3:
            if (nt == 2) GFA_LAUNCH_MFMA(3, 1, false, (MODE == 3 ? 1 : 2));
            else GFA_LAUNCH_MFMA(3, 1, false, 1);
            break;
        default: GFA_LAUNCH_MFMA(4, 1, false, 1); break;
    }
#undef GFA_LAUNCH_MFMA
#undef GFA_LAUNCH_MFMA_L
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_skinny_mfma_bf16(const void* x, const void* w, void* out, int M, int N, int K,
                                    int ldo, int mode, int gate_rows, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0) return (int)hipErrorInvalidValue;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    SkinnyExtra ex = {};
    switch (mode) {
        case 0: return launch_skinny_mfma<0>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
        case 1: return launch_skinny_mfma<1>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
        case 2: return launch_skinny_mfma<2>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
        case 3: return launch_skinny_mfma<3>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
    }
    return (int)hipErrorInvalidValue;
}

// Fused q,k,v projection -> rotary encoding -> q_out and the cache pages, one kernel.
// w [(H + 2 Hkv) hd, K]; head size a multiple of 16, rotary width even, interleaved pairs.
// x [M <= 64, K] are normed rows; or, with ssq_in [t_in, gfa_share_rows(M)], the two halves of
// a norm that gfa_skinny_into_chain_bf16 left (eps the norm's).
extern "C" int gfa_qkv_rope_store_bf16(const void* x, const float* ssq_in, int t_in, float eps,
                                       const void* w, void* q_out, void* k_pages, void* v_pages,
                                       const float* freqs, const int* tok_seq, const int* tok_pos,
                                       const int* table, int table_stride, int M, int K, int H,
                                       int Hkv, int hd, int rot, hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0 || hd % 16 != 0 || rot % 2 != 0 || rot > hd)
        return (int)hipErrorInvalidValue;
    SkinnyExtra ex = {};
    ex.q_out = (bf16_t*)q_out;
    ex.k_pages = (bf16_t*)k_pages;
    ex.v_pages = (bf16_t*)v_pages;
    ex.freqs = freqs;
    ex.tok_seq = tok_seq;
    ex.tok_pos = tok_pos;
    ex.table = table;
    ex.table_stride = table_stride;
    ex.H = H;
    ex.Hkv = Hkv;
    ex.hd = hd;
    ex.rot = rot;
    if (ssq_in) {                                         // second half of a two-kernel norm
        if (t_in <= 0) return (int)hipErrorInvalidValue;
        ex.ssq_in = ssq_in;
        ex.t_in = t_in;
        ex.share_rows = gfa_share_rows(M);
        ex.eps = eps;
        ex.x_pad = ex.share_rows;                         // xg is kept chunked
    }
    const int N = (H + 2 * Hkv) * hd;
    return launch_skinny_mfma<4>((const bf16_t*)x, (const bf16_t*)w, nullptr, M, N, K, 0, 0, ex, stream);
}

// residual [M, N] += x w^T for up to 64 rows, and the first half of the norm that follows:
// xg_out = bfloat16(new residual * next_g), kept chunked ([N / 8][share_rows][8], see
// chunked_elem), ssq_out [tiles, share_rows] = the workgroups' shares of the rows' sums of
// squares, tiles = gfa_skinny_workgroups(2, M, N); share_rows = gfa_share_rows(M).
// N a multiple of 8.  x_chunked: x is kept chunked too (pad gfa_share_rows(M)), as the gate
// of gfa_skinny_after_chain_bf16 leaves its result on request.
extern "C" int gfa_skinny_into_chain_bf16(const void* x, int x_chunked, const void* w,
                                          float* residual, int M, int N, int K, const float* next_g,
                                          void* xg_out, float* ssq_out, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0 || N % 8 != 0 || !next_g || !xg_out || !ssq_out)
        return (int)hipErrorInvalidValue;
    SkinnyExtra ex = {};
    ex.share_rows = gfa_share_rows(M);
    ex.x_pad = x_chunked ? ex.share_rows : 0;
    ex.next_g = next_g;
    ex.xg_out = (bf16_t*)xg_out;
    ex.ssq_out = ssq_out;
    return launch_skinny_mfma<2>((const bf16_t*)x, (const bf16_t*)w, residual, M, N, K, N, 0, ex, stream);
}

// The product that follows: x = xg (M <= 64 rows of K, chunked as the kernel above leaves
// them), the result scaled by rsqrt(sum of ssq_in[:, m] / K + eps), ssq_in [t_in,
// gfa_share_rows(M)].  mode 0 bfloat16 out, 1 float out, 3 gate; out_chunked (gate only, N a
// multiple of 8): the result is left chunked for the product that reads it next.
extern "C" int gfa_skinny_after_chain_bf16(const void* xg, const float* ssq_in, int t_in, float eps,
                                           const void* w, void* out, int M, int N, int K, int ldo,
                                           int mode, int gate_rows, int out_chunked,
                                           hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0 || !ssq_in || t_in <= 0) return (int)hipErrorInvalidValue;
    if (out_chunked && (mode != 3 || N % 8 != 0)) return (int)hipErrorInvalidValue;
    SkinnyExtra ex = {};
    ex.ssq_in = ssq_in;
    ex.t_in = t_in;
    ex.share_rows = gfa_share_rows(M);
    ex.eps = eps;
    ex.x_pad = ex.share_rows;
    ex.out_pad = out_chunked ? ex.share_rows : 0;
    const bf16_t* xp = (const bf16_t*)xg;
    const bf16_t* wp = (const bf16_t*)w;
    switch (mode) {
        case 0: return launch_skinny_mfma<0>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
        case 1: return launch_skinny_mfma<1>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
        case 3: return launch_skinny_mfma<3>(xp, wp, out, M, N, K, ldo, gate_rows, ex, stream);
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
