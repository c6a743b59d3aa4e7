// Products of 17..64 rows of x with a weight matrix that is kept a second time in the order
// in which the matrix cores read it: out = x W^T, x [M <= 64, K] row-major bfloat16, W [N, K].
//
// "Tiled" W: [ceil(N / 16)][Kp / 8][16][8] bfloat16 with Kp = K rounded up to 128 (zeros
// beyond N and K).  A tile is 16 rows of W; the A operand of v_mfma_f32_16x16x32_bf16 for 32
// values of k of a tile (lane l: row l % 16, k = 8 (l / 16) .. +7) is 1 KB of consecutive bytes
// with lane l at byte 16 l.  A wave therefore loads its weights straight into operand
// registers, 16 bytes per lane and 1 KB per instruction, and W never passes through LDS.
//
// With this many rows, what a compute unit has to take in per byte of W is no longer W alone:
// every 16 rows of W meet all rows of x.  So the waves of a workgroup (4 to 16, one tile of W
// each) walk the same range of k together and share x through LDS: per 128 values of k, the
// workgroup copies CT * 16 rows x 256 bytes of x into one of three stages once, and every wave
// reads its B operands from there.  A compute unit takes in about 15 bytes per clock whatever
// their source, so the bytes of x per byte of W (CT tiles of rows per wave's tile of W) and the number of compute
// units that have a workgroup decide the rate: the launcher picks waves per workgroup and
// slices of K so that the workgroups just fill the compute units.
//
// x is requested by instructions the compiler cannot move or remove (written as asm): it sinks
// ordinary loads to their use, behind the weight loads, and loads return in order.  Their wait
// is counted by hand: four weight loads follow them in every step of the main loop.  The last
// steps request nothing and wait for everything.
//
// Epilogues (MODE): 1 float [M, ldo]; 3 gate, for a matrix whose tiles
// hold eight rows of W1 and the eight rows of W3 that belong to the same columns: out[m, n] =
// silu(x W1[n]) * (x W3[n]) in bfloat16 (model.py:227); 5 float partial sums [slices, M, N] of
// a product whose K is cut into slices (added in slice order by the kernels of
// gemm_wide_bf16.hip).
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

#define TL_PIECE 128                       // values of k per step
#define TL_ROW_BYTES (TL_PIECE * 2)        // of a row of x in a stage
#define TL_W_PIECE (16 * TL_PIECE * 2)     // bytes of a tile of W per step: 4 KB

#define TL_XLOAD(dst, ptr) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory")
// All but the newest N loads have arrived.  The wait names the registers that the asm loads
// fill: what reads them is thereby ordered behind it (a register move or select is no memory
// access, and the compiler would else be free to schedule it before the wait).
#define TL_ARRIVED(N, R)                                                                         \
    asm volatile("s_waitcnt vmcnt(" #N ")" : "+v"(R.a), "+v"(R.b), "+v"(R.c), "+v"(R.d) : : "memory")

__device__ __forceinline__ float tl_silu(float a) { return a / (1.f + expf(-a)); }

template <int NWAVES, int CT, int MODE>
__global__ __launch_bounds__(NWAVES * 64) void tiled_kernel(
        const bf16_t* __restrict__ x, const bf16_t* __restrict__ wt, void* __restrict__ out, int M,
        int N, int K, int ldo, int pieces_per_slice) {
    constexpr int STAGE = CT * 16 * TL_ROW_BYTES;                    // a piece of x: CT * 4 KB
    constexpr int ITEMS = STAGE / 16;                                // 16-byte items of a stage
    constexpr int XC = (ITEMS + NWAVES * 64 - 1) / (NWAVES * 64);    // items per thread
    static_assert(XC <= 4, "a stage of x is copied in at most four rounds");
    __shared__ __attribute__((aligned(16))) char xs[3][STAGE];       // piece p of x in stage p % 3
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int fi = lane & 15, fg = lane >> 4;
    const int n_tiles = (N + 15) >> 4;
    const int tile = blockIdx.x * NWAVES + wave;                     // 16 rows of W
    const int tile_c = tile < n_tiles ? tile : n_tiles - 1;          // waves beyond the matrix walk along
    const int P = (K + TL_PIECE - 1) / TL_PIECE;
    const int p0 = blockIdx.y * pieces_per_slice;
    int p1 = p0 + pieces_per_slice;
    if (p1 > P) p1 = P;
    const int np = p1 - p0;                                          // the launcher leaves no slice empty
    const char* wbase = (const char*)wt + ((size_t)tile_c * P + p0) * TL_W_PIECE + lane * 16;

    // x: item i of a stage is row i / 16, 16-byte chunk i % 16; in LDS the chunk is kept at
    // position chunk ^ (row % 16), so that neither the copy (sixteen lanes: one row, sixteen
    // chunks) nor an operand read (sixteen lanes: sixteen rows, one chunk) meets a bank twice
    const char* xsrc[4];
    int xdst[4];
    bool xlive[4];
    const int k_chunks = K >> 3;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int item = (int)threadIdx.x + i * NWAVES * 64;
        xlive[i] = i < XC && item < ITEMS;
        const int row = xlive[i] ? item >> 4 : 0, chunk = item & 15;
        const int m = row < M ? row : M - 1;                         // rows beyond M: any finite data
        xsrc[i] = (const char*)(x + (size_t)m * K);                  // the row; the chunk is added per piece
        xdst[i] = row * TL_ROW_BYTES + ((chunk ^ (row & 15)) << 4);
    }
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    struct XR { u32x4 a, b, c, d; bool inside; };
    auto load_x = [&](int p, XR& r) {
        // a chunk beyond K (the last piece of a K that is no multiple of 128) meets zeros of the
        // tiled W, but zero times whatever lies there may be no number: such a chunk is read
        // from the row's start and written as zeros
        const int pc = p < np ? p : np - 1;
        const int kc = (p0 + pc) * (TL_PIECE / 8) + ((int)threadIdx.x & 15);
        r.inside = kc < k_chunks;
        const size_t off = r.inside ? (size_t)kc * 16 : 0;
        r.b = r.c = r.d = u32x4{0, 0, 0, 0};                         // those that no load fills
        TL_XLOAD(r.a, xsrc[0] + off);
        if (XC > 1) TL_XLOAD(r.b, xsrc[1] + off);
        if (XC > 2) TL_XLOAD(r.c, xsrc[2] + off);
        if (XC > 3) TL_XLOAD(r.d, xsrc[3] + off);
    };
    auto write_x = [&](char* stage, const XR& r) {
        const u32x4 zero = {0, 0, 0, 0};
        // sixteen waves have more threads than a stage of two row tiles has items
        if (xlive[0]) *(u32x4*)(stage + xdst[0]) = r.inside ? r.a : zero;
        if (XC > 1 && xlive[1]) *(u32x4*)(stage + xdst[1]) = r.inside ? r.b : zero;
        if (XC > 2 && xlive[2]) *(u32x4*)(stage + xdst[2]) = r.inside ? r.c : zero;
        if (XC > 3 && xlive[3]) *(u32x4*)(stage + xdst[3]) = r.inside ? r.d : zero;
    };

    floatx4_t acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[ct] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    uint4 wr[3][4];                                                  // the ring of W: piece p in wr[p % 3]
    auto load_w = [&](int p, uint4 (&r)[4]) {
        const char* src = wbase + (size_t)(p < np ? p : np - 1) * TL_W_PIECE;
#pragma unroll
        for (int s = 0; s < 4; ++s) r[s] = stream_load16(src + s * 1024);
    };
    auto multiply = [&](const char* st, const uint4 (&r)[4]) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bf16x8_t a = __builtin_bit_cast(bf16x8_t, r[s]);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const uint4 bu = *(const uint4*)(st + (ct * 16 + fi) * TL_ROW_BYTES + (((s * 4 + fg) ^ fi) << 4));
                acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8_t, bu), acc[ct], 0, 0, 0);
            }
        }
    };
    {
        XR r0, r1;
        load_x(0, r0);
        load_w(0, wr[0]);
        load_x(1, r1);
        load_w(1, wr[1]);
        load_w(2, wr[2]);
        TL_ARRIVED(0, r0);
        TL_ARRIVED(0, r1);
        write_x(xs[0], r0);
        write_x(xs[1], r1);
    }
    // step p: barrier; request x(p + 2); multiply piece p; request W(p + 3); x(p + 2) into the
    // stage that piece p - 1 was read from (every wave is past the barrier, so past that read)
#define TL_STEP(PIECE, S)                                                                        \
    {                                                                                            \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                       \
        __builtin_amdgcn_s_barrier();                                                            \
        asm volatile("" ::: "memory");                                                           \
        XR r;                                                                                    \
        load_x((PIECE) + 2, r);                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        multiply(xs[S], wr[S]);                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        load_w((PIECE) + 3, wr[S]);                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        TL_ARRIVED(4, r);                                    /* the four loads of W stay out */   \
        write_x(xs[((S) + 2) % 3], r);                                                           \
    }
    // Whole trips of three only.  A trip that could end early would leave paths into the loop's
    // head on which the newest loads are those of the first ring entry, and the compiler would
    // wait for everything there; and in steps behind the loop the weight loads, whose values
    // nothing reads, are removed, so the counted wait above would count wrongly.
    int pb = 0;
    for (; pb + 3 <= np; pb += 3) {
        TL_STEP(pb, 0)
        TL_STEP(pb + 1, 1)
        TL_STEP(pb + 2, 2)
    }
#undef TL_STEP
    // the last one or two pieces: requested already; nothing more is
#define TL_LAST(S)                                                                               \
    {                                                                                            \
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                              \
        __builtin_amdgcn_s_barrier();                                                            \
        asm volatile("" ::: "memory");                                                           \
        multiply(xs[S], wr[S]);                                                                  \
    }
    if (pb < np) TL_LAST(0)
    if (pb + 1 < np) TL_LAST(1)
#undef TL_LAST
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                 // requests of the last steps
    if (tile >= n_tiles) return;

    // lane l holds rows 4 (l / 16) .. +3 of the tile (columns of out) for x row l % 16 of each tile of rows
    if (MODE == 3) {
        // rows 0..7 of the tile are W1's, rows 8..15 W3's for the same eight columns: the lanes
        // of the lower half get their partner's value from the lane 32 above
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float up[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) up[j] = __shfl(acc[ct][j], (lane + 32) & 63, GFA_WAVE);
            const int m = ct * 16 + fi, n = tile * 8 + fg * 4, cols = N >> 1;     // N counts W1's and W3's rows
            if (fg < 2 && m < M) {
                bf16_t* o = (bf16_t*)out + (size_t)m * ldo + n;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (n + j < cols) o[j] = float_to_bf16(tl_silu(acc[ct][j]) * up[j]);
            }
        }
        return;
    }
    const int n = tile * 16 + fg * 4;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int m = ct * 16 + fi;
        if (m >= M) continue;
        if (MODE == 5) {
            float* o = (float*)out + ((size_t)blockIdx.y * M + m) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(floatx4_t*)o = acc[ct];
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (n + j < N) o[j] = acc[ct][j];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (n + j >= N) continue;
                if (MODE == 1) ((float*)out)[(size_t)m * ldo + n + j] = acc[ct][j];
                else ((bf16_t*)out)[(size_t)m * ldo + n + j] = float_to_bf16(acc[ct][j]);
            }
        }
    }
}

static int tl_compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        hipGetDevice(&dev);
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        cus = n > 0 ? n : 1;
    }
    return cus;
}

// Waves per workgroup and slices of K for a product with `tiles` tiles of W and `pieces`
// steps of k.  In units of 4 KB that a compute unit takes in: a workgroup of nw waves takes
// nw + 4 per step (its tiles of W and four tiles of rows of x), the workgroups go over the
// compute units in rounds, and a sliced product writes and reads 2 * slices * tiles units of
// partial sums, which cost about three times as much as streamed weights.  This fits what was
// measured on 256 compute units at 64 rows (28672 x 4096: 42.8 us with 7 waves, 256
// workgroups, against 46.5 with 8 and 50.9 with 4; 4096 x 14336: 23.8 us with 8 waves and 8
// slices against 28.7 with 16 and 16; 4096 x 4096: 11.5 us with 4 waves and 4 slices; 6144 x
// 4096: 13.1 us with 6 waves and 4 slices against 16.1 with 8 and 4).
static const int TL_WAVES[] = {16, 12, 8, 7, 6, 4};

static void tl_plan(int tiles, int pieces, bool may_slice, int* nw_out, int* slices_out) {
    const int cus = tl_compute_units();
    int best_nw = 8, best_s = 1;
    double best_cost = 1e30;
    for (int nw : TL_WAVES) {
        const int groups = (tiles + nw - 1) / nw;
        const int most = may_slice && pieces >= 8 ? pieces / 4 : 1;  // a slice keeps four steps at least
        for (int s = 1; s <= most && s <= 64; ++s) {
            const long rounds = ((long)groups * s + cus - 1) / cus;
            const int per = (pieces + s - 1) / s;
            const double cost = (double)rounds * per * (nw + 4) + (s > 1 ? 6.0 * s * tiles / cus : 0.0);
            if (cost < best_cost - 1e-9) {
                best_cost = cost;
                best_nw = nw;
                best_s = s;
            }
        }
    }
    *nw_out = best_nw;
    *slices_out = best_s;
}

// Slices the launcher cuts K into for this shape (the partial sums are [slices, M, N]).
extern "C" int gfa_tiled_slices(int N, int K, int mode) {
    int nw, s;
    tl_plan((N + 15) / 16, (K + TL_PIECE - 1) / TL_PIECE, mode == 5, &nw, &s);
    return s;
}

template <int MODE>
static int launch_tiled(const bf16_t* x, const bf16_t* wt, void* out, int M, int N, int K, int ldo,
                        hipStream_t stream) {
    const int tiles = (N + 15) / 16, pieces = (K + TL_PIECE - 1) / TL_PIECE;
    int nw, slices;
    tl_plan(tiles, pieces, MODE == 5, &nw, &slices);
    const int per = (pieces + slices - 1) / slices;
    slices = (pieces + per - 1) / per;                               // no empty slice
    const dim3 grid((tiles + nw - 1) / nw, slices);
    // tiles of sixteen rows of x per wave: two up to 32 rows, else four
#define TL_LAUNCH(NW, CTV) tiled_kernel<NW, CTV, MODE><<<grid, NW * 64, 0, stream>>>(x, wt, out, M, N, K, ldo, per)
#define TL_LAUNCH_NW(CTV)                                                                        \
    switch (nw) {                                                                                \
        case 4: TL_LAUNCH(4, CTV); break;                                                        \
        case 6: TL_LAUNCH(6, CTV); break;                                                        \
        case 7: TL_LAUNCH(7, CTV); break;                                                        \
        case 8: TL_LAUNCH(8, CTV); break;                                                        \
        case 12: TL_LAUNCH(12, CTV); break;                                                      \
        default: TL_LAUNCH(16, CTV); break;                                                      \
    }
    if (M <= 32) TL_LAUNCH_NW(2) else TL_LAUNCH_NW(4)
#undef TL_LAUNCH_NW
#undef TL_LAUNCH
    return GFA_LAUNCH_RESULT();
}

// x [M <= 64, K] row-major, wt the tiled form of W [N, K] (gate mode: of [2 N, K] with tiles of
// eight and eight rows, N = the gate's columns), K a multiple of 8.  out: [M, ldo] bfloat16
// (mode 3) or float (mode 1), or the float partial sums [gfa_tiled_slices(N, K, 5), M, N]
// (mode 5).
extern "C" int gfa_tiled_bf16(const void* x, const void* wt, void* out, int M, int N, int K, int ldo,
                              int mode, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 != 0) return (int)hipErrorInvalidValue;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)wt;
    switch (mode) {
        case 1: return launch_tiled<1>(xp, wp, out, M, N, K, ldo, stream);
        // the gate's tiles hold eight columns each: twice as many tiles as columns / 16
        case 3: return launch_tiled<3>(xp, wp, out, M, 2 * N, K, ldo, stream);
        case 5: return launch_tiled<5>(xp, wp, out, M, N, K, ldo, stream);
    }
    return (int)hipErrorInvalidValue;
}

// W [N, K] row-major -> its tiled form [ceil(N / 16)][Kp / 8][16][8], Kp = K rounded up to 128,
// zeros beyond N and K.  gate_rows > 0: W is [2 gate_rows, K], rows of W1 then rows of W3, and
// tile t holds rows 8 t .. 8 t + 7 of W1 followed by the same rows of W3 (zeros beyond
// gate_rows).  One thread per 16-byte chunk of the result.
__global__ __launch_bounds__(256) void tile_weights_kernel(const bf16_t* __restrict__ w,
                                                           bf16_t* __restrict__ wt, int N, int K,
                                                           int gate_rows, size_t chunks) {
    const size_t c = blockIdx.x * (size_t)256 + threadIdx.x;
    if (c >= chunks) return;
    const int Kp8 = ((K + TL_PIECE - 1) / TL_PIECE) * (TL_PIECE / 8);
    const int r = (int)(c & 15);
    const size_t rest = c >> 4;
    const int kc = (int)(rest % Kp8);
    const int tile = (int)(rest / Kp8);
    long row;
    if (gate_rows > 0) {
        const int col = tile * 8 + (r & 7);
        row = col < gate_rows ? (long)col + (r >= 8 ? gate_rows : 0) : -1;
    } else {
        row = tile * 16 + r;
        if (row >= N) row = -1;
    }
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row >= 0 && kc * 8 < K) v = *(const uint4*)(w + (size_t)row * K + (size_t)kc * 8);
    *(uint4*)(wt + c * 8) = v;
}

// Elements of the tiled form of a matrix of `rows` rows (gate: 2 * gate_rows) and K columns.
extern "C" size_t gfa_tiled_elements(int rows, int K, int gate_rows) {
    const size_t tiles = gate_rows > 0 ? (size_t)(gate_rows + 7) / 8 : (size_t)(rows + 15) / 16;
    const size_t Kp = (size_t)((K + TL_PIECE - 1) / TL_PIECE) * TL_PIECE;
    return tiles * 16 * Kp;
}

extern "C" int gfa_tile_weights(const void* w, void* wt, int N, int K, int gate_rows,
                                hipStream_t stream) {
    if (N <= 0 || K <= 0 || K % 8 != 0 || (gate_rows > 0 && N != 2 * gate_rows))
        return (int)hipErrorInvalidValue;
    const size_t chunks = gfa_tiled_elements(N, K, gate_rows) / 8;
    const size_t blocks = (chunks + 255) / 256;
    if (blocks > 0x7fffffffu) return (int)hipErrorInvalidValue;
    tile_weights_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)w, (bf16_t*)wt, N, K,
                                                              gate_rows, chunks);
    return GFA_LAUNCH_RESULT();
}
