// Attention over the paged cache on the matrix cores, for prompts and for single tokens.
//
// One wavefront owns up to 16 * RT query rows of one sequence and one key/value head; a
// row is a (token, query head of that kv head's group) pair, heads fastest, so the keys
// and values of a group are read once for all its query heads (the reference expands
// them with repeat_interleave instead, model.py:209-210).  The wave walks the keys in
// blocks of 32 with a running maximum and sum per row (all in float), and never reads a
// key beyond its rows' positions: the causal mask of model.py:134,138 is the loop bound
// plus a comparison inside the last blocks.
//
// Both products are formed transposed, so that every operand is read in the layout the
// cache already has and the probabilities never leave their registers:
//   S^T = K Q^T    A = 16 keys x 32 dims from a key page (rows [64, hd]),
//                  B = Q^T from registers;  lane l gets keys 4 (l / 16) .. +3 of row l % 16.
//   O^T = V^T P^T  A = 16 dims x 32 keys from a value page (transposed, [hd, 64]),
//                  B = P^T: exactly the 8 probabilities the lane just computed, when the
//                  32 keys of a block are numbered (16-key tile, 4 (l / 16) .. +3) per lane.
// v_mfma_f32_16x16x32_bf16: lane l supplies row (A) / column (B) l % 16, k = 8 (l / 16) .. +7,
// and receives rows 4 (l / 16) .. +3 of column l % 16.
//
// For single-token steps the context of one (sequence, kv head) is split over several
// waves; each writes an unnormalised partial result with its maximum and sum, and a
// second kernel combines them in split order.
#include "common.h"
#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

union Frag {
    uint4 u;
    uint2 h[2];
    bf16_t e[8];
    bf16x8_t v;
};

#define LOG2E 1.4426950408889634f

// Maximum (sum) over the four lanes i, i + 16, i + 32, i + 48: the lanes that hold one row's
// scores.  The swaps exchange rows of sixteen lanes between two registers (odd rows of the
// first with even rows of the second; the upper half of the first with the lower half of the
// second), so two copies of a value meet their neighbours without a trip through LDS.
__device__ __forceinline__ float max_over_lane_groups(float v) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float sum_over_lane_groups(float v) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// SINGLE: every sequence brings exactly one token and a kv head's group fits one 16-row tile.
// The grid is then (splits, kv heads, sequences) and nothing in the kernel's first round of
// loads depends on another load: the query rows (row of sequence s = s), the sequence's
// position and the first 63 entries of its page row - one per lane, handed out by readlane
// as the blocks come - are requested together, and the keys and values follow in the second
// round.  Otherwise q_start -> position -> page number -> keys is a chain of four.
// SLICED (with SINGLE): the step's q, k and v rows are not there yet - only the float partial
// sums [S, sequences, (H + 2 Hkv) * hd] of the sliced product that makes them.  The workgroup
// adds the slices of its own sequence and kv head (the group's query heads, the new key, the
// new value), rotates queries and key by the token's position (interleaved pairs, the
// arithmetic of rope_cache_sliced_bf16x8_kernel in core.hip) and keeps them in LDS: the
// queries become its operand, the key and value are put into the operands of the block that
// holds the token's position after that block's loads, and the workgroup of the last split
// writes them to the cache for the steps to come.  The rotation and cache-write kernel and
// its round trip through memory fall away.
struct SlicedRowsIn {
    const float* part;        // null unless SLICED
    int S;
    size_t slice;             // elements between slices
    int width;                // (H + 2 Hkv) * hd
    const float* freqs;       // [rot / 2], null if rot == 0
    int rot;
    bf16_t* k_out;            // the caches again, to write to
    bf16_t* v_out;
};
#define SL_MAX_ROT 256
#define SL_MAX_ELEMS (18 * 128)           // sixteen query heads, key, value of up to 128 dims

template <int DS, int RT, bool PREFETCH, bool SINGLE = false, bool SLICED = false>
__global__ __launch_bounds__(RT == 1 ? 512 : 256) void attention_mfma_kernel(
        const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
        const bf16_t* __restrict__ v_pages, const int* __restrict__ q_start,
        const int* __restrict__ start_pos, const int* __restrict__ table, int table_stride,
        bf16_t* __restrict__ out, float* __restrict__ ws_o, float* __restrict__ ws_ml, int H,
        int Hkv, int hd, float scale_log2, int window, int n_splits, int total_rows, int out_pad,
        SlicedRowsIn sl) {
    constexpr int DT = DS * 2;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    static_assert(!SINGLE || RT == 1, "one token per sequence is one tile of rows");
    static_assert(!SLICED || SINGLE, "partial sums are taken for one token per sequence");
    __shared__ float sl_cs[SLICED ? SL_MAX_ROT : 1];                             // cos, sin per pair
    __shared__ __attribute__((aligned(16))) bf16_t sl_rows[SLICED ? SL_MAX_ELEMS : 8];   // q heads, k, v
    const int lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    // SINGLE: lane i < 63 holds entry i of the page row and lane 63 the sequence's position,
    // from one load instruction that needs only arguments which arrive in registers; it is
    // issued before anything waits for the arguments that are loaded
    int first_pages = 0;
    if (SINGLE) {
        const int* row = table + (size_t)blockIdx.z * table_stride;
        const int* src = lane == 63 ? start_pos + blockIdx.z : row + (lane < table_stride ? lane : table_stride - 1);
        first_pages = *src;
        __builtin_amdgcn_sched_barrier(0);
    }
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int g = blockIdx.y;
    const int R = H / Hkv;
    int seq, split, q0, rows_total, row0;
    if (SINGLE) {
        seq = blockIdx.z;
        split = blockIdx.x;
        q0 = seq;
        rows_total = R;
        row0 = 0;
    } else {
        seq = blockIdx.z / n_splits;
        split = blockIdx.z - seq * n_splits;
        q0 = q_start[seq];
        rows_total = (q_start[seq + 1] - q0) * R;
        row0 = blockIdx.x * 16 * RT;
        if (row0 >= rows_total) return;                  // the whole workgroup leaves
    }
    const int* pages = table + (size_t)seq * table_stride;
    const int spos = SINGLE ? __builtin_amdgcn_readlane(first_pages, 63) : start_pos[seq];

    if (SLICED) {
        // four elements at a time: R query heads of this group, then the key, then the value.
        // A thread's first four are requested before the table of cosines and sines is made
        // (their addresses need no position), so the two round trips overlap.
        const int per_head = hd >> 2, n_items = (R + 2) * per_head;
        const float* row = sl.part + (size_t)seq * sl.width;
        auto column = [&](int i) {
            const int head = i / per_head, d = (i - head * per_head) * 4;
            return (head < R ? g * R + head : head == R ? H + g : H + Hkv + g) * hd + d;
        };
        auto summed = [&](int i) {
            const int col = column(i);
            float4 a = *(const float4*)(row + col);
            for (int sidx = 1; sidx < sl.S; ++sidx) {
                const float4 b = *(const float4*)(row + (size_t)sidx * sl.slice + col);
                a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
            }
            return a;
        };
        auto rotate_and_keep = [&](int i, float4 a) {
            const int head = i / per_head, d = (i - head * per_head) * 4;
            if (head <= R && d < sl.rot) {
                const float c0 = sl_cs[d], s0 = sl_cs[d + 1], c1 = sl_cs[d + 2], s1 = sl_cs[d + 3];
                a = make_float4(a.x * c0 - a.y * s0, a.y * c0 + a.x * s0,
                                a.z * c1 - a.w * s1, a.w * c1 + a.z * s1);
            }
            union { uint2 u; bf16_t e[4]; } w;
            w.e[0] = float_to_bf16(a.x); w.e[1] = float_to_bf16(a.y);
            w.e[2] = float_to_bf16(a.z); w.e[3] = float_to_bf16(a.w);
            *(uint2*)(sl_rows + head * hd + d) = w.u;
        };
        const int first = threadIdx.x;
        float4 a_first = make_float4(0.f, 0.f, 0.f, 0.f);
        if (first < n_items) a_first = summed(first);
        for (int i = threadIdx.x; i < sl.rot / 2; i += blockDim.x)
            sincosf((float)spos * sl.freqs[i], &sl_cs[2 * i + 1], &sl_cs[2 * i]);
        __syncthreads();
        if (first < n_items) rotate_and_keep(first, a_first);
        for (int i = first + blockDim.x; i < n_items; i += blockDim.x) rotate_and_keep(i, summed(i));
        __syncthreads();
        if (split == n_splits - 1 && wave == 0 && sl.k_out) {
            // the new key and value go to their place in the cache (the reads of this step
            // take them from LDS: this write need not have landed)
            const int pi = spos >> 6, off = spos & (GFA_PAGE - 1);
            const int page = pi < 63 ? __builtin_amdgcn_readlane(first_pages, pi < 63 ? pi : 0) : pages[pi];
            if (lane < (hd >> 3))
                *(uint4*)(sl.k_out + key_elem(page, g, off, lane * 8, Hkv, hd)) = *(const uint4*)(sl_rows + R * hd + lane * 8);
            for (int d = lane; d < hd; d += 64)
                sl.v_out[value_elem(page, g, d, off, Hkv, hd)] = sl_rows[(R + 1) * hd + d];
        }
    }

    Frag qf[RT][DS];
    int rpos[RT];             // position of this lane's row in tile rt, -1 if there is none
    size_t orow[RT];          // (token, head) index of that row in q / out
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int r = row0 + rt * 16 + li;
        const bool valid = r < rows_total;
        const int t = (valid && !SINGLE) ? r / R : 0, hh = valid ? r - t * R : 0;
        rpos[rt] = valid ? spos + t : -1;
        orow[rt] = (size_t)(q0 + t) * H + g * R + hh;
        const bf16_t* qrow = SLICED ? sl_rows + hh * hd : q + orow[rt] * hd;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int d = ds * 32 + lg * 8;
            qf[rt][ds].u = (valid && d < hd) ? *(const uint4*)(qrow + d) : make_uint4(0, 0, 0, 0);
        }
    }
    const int last_row = (row0 + 16 * RT - 1 < rows_total - 1) ? row0 + 16 * RT - 1 : rows_total - 1;
    const int pmin = SINGLE ? spos : spos + row0 / R, pmax = SINGLE ? spos : spos + last_row / R;
    const int lo = (window > 0 && pmin - window + 1 > 0) ? pmin - window + 1 : 0;
    const int kb_lo = lo >> 5, nkb = (pmax >> 5) - kb_lo + 1;
    // 32-bit: a sequence has at most table_stride * 2 blocks, the host checks that times splits
    const int kb_begin = kb_lo + (int)((unsigned)(split * nkb) / (unsigned)n_splits);
    const int kb_end = kb_lo + (int)((unsigned)((split + 1) * nkb) / (unsigned)n_splits);

    float m[RT], l[RT];
    floatx4_t o[RT][DT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[rt][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    // Row r of key tile kt stands for key 8 (r / 4) + 4 kt + r % 4 of the block, so that the
    // eight scores a lane holds (rows 4 lg .. +3 of both tiles) belong to the eight
    // consecutive keys 8 lg .. +7 and its value operand is one 16-byte load.  The cache keeps
    // keys and values in this order (common.h):
    // keys: tile kt, row li -> slot 16 kt + li of the block, dims ds * 32 + lg * 8 .. +7
    // values: dims dt * 16 + li, keys 8 lg .. +7 of the block
    auto load_block = [&](int kb, Frag (&kf)[2][DS], Frag (&vf)[DT]) {
        int page;
        if (SINGLE && (kb >> 1) < 63) page = __builtin_amdgcn_readlane(first_pages, kb >> 1);
        else page = pages[kb >> 1];
        // Every lane loads; for dims beyond the head it is chunk 0 or tile 0, which meets zeros
        // in the query's operand or goes into accumulators that are never stored.  No load
        // runs under a branch or a partial execution mask (a choice between the loaded value
        // and zero would be turned into one), so the waits can count requests.  In the
        // cache's layout a load instruction reads consecutive lines: 4 x 256 bytes of keys
        // (16 slots of a chunk each), 1 KB of values.
        const bf16_t* kbase = k_pages + cache_region(page, g, Hkv, hd) + (size_t)(kb & 1) * 32 * hd;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) {
                const int d = ds * 32 + lg * 8;
                kf[kt][ds].u = *(const uint4*)(kbase + (d < hd ? d >> 3 : 0) * 256 + (kt * 16 + li) * 8);
            }
        const bf16_t* vbase = v_pages + cache_region(page, g, Hkv, hd) + (kb & 1) * 512 + lane * 8;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            vf[dt].u = *(const uint4*)(vbase + (dt * 16 < hd ? dt : 0) * 1024);
    };
    auto compute_block = [&](int kb, Frag (&kf)[2][DS], Frag (&vf)[DT]) {
        const int key0 = kb * 32 + lg * 8;                 // this lane's keys: key0 .. key0 + 7
        if (SLICED && kb == (pmax >> 5)) {
            // the block of the token itself: its key and value come from LDS, whatever the
            // cache held at their place when the block was loaded
            const int in_block = pmax & 31, slot = key_slot(in_block);
            if (li == (slot & 15)) {
#pragma unroll
                for (int ds = 0; ds < DS; ++ds) {
                    const int d = ds * 32 + lg * 8;
                    if (d < hd) {
                        const uint4 knew = *(const uint4*)(sl_rows + R * hd + d);
                        if (slot >> 4) kf[1][ds].u = knew; else kf[0][ds].u = knew;
                    }
                }
            }
            if (lg == (in_block >> 3)) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16_t vnew = sl_rows[(R + 1) * hd + (dt * 16 < hd ? dt * 16 : 0) + li];
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (e == (in_block & 7)) vf[dt].e[e] = vnew;
                }
            }
        }
        floatx4_t s[RT][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                s[rt][kt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < DS; ++ds)
                    s[rt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kt][ds].v, qf[rt][ds].v, s[rt][kt], 0, 0, 0);
            }
        if (kb * 32 + 31 > pmax) {          // slots beyond the newest key hold no data yet
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (key0 + e > pmax) vf[dt].e[e] = 0;
        }
        // blocks wholly below every row's position (and inside every window) need no mask
        const bool masked = kb * 32 + 31 > pmin || (window > 0 && kb * 32 < pmax - window + 1);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            // raw scores; the scale is positive, so it is applied to the maximum and inside
            // the exponent's multiply-add instead of to every score
            float sv[8];
            float mx = -INFINITY;
            if (masked) {
                const int first = (window > 0) ? rpos[rt] - window + 1 : 0;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = key0 + e;
                    sv[e] = (key <= rpos[rt] && key >= first) ? s[rt][e >> 2][e & 3] : -INFINITY;
                    mx = fmaxf(mx, sv[e]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    sv[e] = s[rt][e >> 2][e & 3];
                    mx = fmaxf(mx, sv[e]);
                }
            }
            mx = max_over_lane_groups(mx) * scale_log2;
            const float m_new = fmaxf(m[rt], mx);
            // a row without any key so far keeps m = -inf: exp2(-inf - -inf) must not be formed
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m[rt] - m_safe);
            Frag pf;
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sv[e], scale_log2, -m_safe));   // 2^-inf = 0
                sum += p;
                pf.e[e] = float_to_bf16(p);
            }
            l[rt] = l[rt] * alpha + sum;
            m[rt] = m_new;
            // the running maximum rarely moves after the first blocks: skip the rescale then
            // (a real branch: as a choice per element it costs as much as the rescale)
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
                asm volatile("" ::: "memory");
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[rt][dt] *= alpha;
            }
#pragma unroll
            // every tile of dims is multiplied, also those beyond the head (their results are
            // never stored).  A test of the head size here (`if (dt * 16 < hd)`) ends a basic
            // block directly behind a matrix instruction, and for the block it jumps to the
            // compiler once left out the wait states that the instruction's result needs: on
            // the path head size 16 takes, the accumulator was copied back
            // (v_accvgpr_read_b32) three wait states after the instruction instead of seven,
            // and one of a lane's four sums of the first row tile lost the block's product.
            // Straight-line code gets its waits; tests/test_isa_hazards.py reads the compiled
            // kernels for such sequences.
            for (int dt = 0; dt < DT; ++dt)
                o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf.v, o[rt][dt], 0, 0, 0);
        }
    };

    // the waves of a workgroup take the blocks of their share in turn
    int kb = kb_begin + wave;
    if (PREFETCH) {
        Frag kfa[2][DS], vfa[DT], kfb[2][DS], vfb[DT];
        if (kb < kb_end) load_block(kb, kfa, vfa);
        for (; kb < kb_end; kb += 2 * nw) {
            const bool more = kb + nw < kb_end;
            if (more) load_block(kb + nw, kfb, vfb);
            compute_block(kb, kfa, vfa);
            if (more) {
                if (kb + 2 * nw < kb_end) load_block(kb + 2 * nw, kfa, vfa);
                compute_block(kb + nw, kfb, vfb);
            }
        }
    } else if (SINGLE) {
        // Two blocks in flight: a block's keys and values are requested before the block
        // ahead of it is multiplied.  Every load is issued unconditionally - a block beyond
        // the wave's share stands for the share's last one (or the context's first) and is
        // not multiplied - so that the waits count requests instead of draining them all.
        Frag kfa[2][DS], vfa[DT], kfb[2][DS], vfb[DT];
        const int kb_safe = kb_end > kb_lo ? kb_end - 1 : kb_lo;
        load_block(kb < kb_end ? kb : kb_safe, kfa, vfa);
        for (; kb < kb_end; kb += 2 * nw) {
            load_block(kb + nw < kb_end ? kb + nw : kb_safe, kfb, vfb);
            compute_block(kb, kfa, vfa);
            load_block(kb + 2 * nw < kb_end ? kb + 2 * nw : kb_safe, kfa, vfa);
            if (kb + nw < kb_end) compute_block(kb + nw, kfb, vfb);
        }
    } else {
        Frag kfa[2][DS], vfa[DT];
        for (; kb < kb_end; kb += nw) {
            load_block(kb, kfa, vfa);
            compute_block(kb, kfa, vfa);
        }
    }

    float lt[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        lt[rt] = sum_over_lane_groups(l[rt]);
    }
    if (nw > 1) {                 // the waves' partial results meet in LDS, added in wave order
        float* sm_ml = (float*)smem;                                  // [nw - 1][RT][16][2]: waves 1 ..
        floatx4_t* sm_o = (floatx4_t*)(smem + (size_t)(nw - 1) * RT * 16 * 2 * sizeof(float));
        if (wave > 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if (lg == 0) {
                    sm_ml[(((wave - 1) * RT + rt) * 16 + li) * 2] = m[rt];
                    sm_ml[(((wave - 1) * RT + rt) * 16 + li) * 2 + 1] = lt[rt];
                }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) sm_o[(((wave - 1) * RT + rt) * DT + dt) * 64 + lane] = o[rt][dt];
            }
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < nw; ++w)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float mw = sm_ml[(((w - 1) * RT + rt) * 16 + li) * 2];
                if (mw == -INFINITY) continue;
                const float lw = sm_ml[(((w - 1) * RT + rt) * 16 + li) * 2 + 1];
                const float m_new = fmaxf(m[rt], mw);
                const float a = __builtin_amdgcn_exp2f(m[rt] - m_new);     // 0 if this wave saw no key
                const float b = __builtin_amdgcn_exp2f(mw - m_new);
                lt[rt] = lt[rt] * a + lw * b;
                m[rt] = m_new;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    o[rt][dt] = o[rt][dt] * a + sm_o[(((w - 1) * RT + rt) * DT + dt) * 64 + lane] * b;
            }
    }

#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rpos[rt] < 0) continue;
        if (n_splits == 1) {
            const float inv = 1.f / lt[rt];
            // out_pad (SINGLE only): the result is left chunked (common.h) for the product
            // that reads it next; the row is the token, the column (head, dim)
            const int tok = SINGLE ? seq : 0, col0 = SINGLE ? (int)(orow[rt] - (size_t)seq * H) * hd : 0;
            bf16_t* orow_p = out + orow[rt] * hd;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 16 + lg * 4;
                if (d < hd) {
                    Frag w;
#pragma unroll
                    for (int j = 0; j < 4; ++j) w.e[j] = float_to_bf16(o[rt][dt][j] * inv);
                    bf16_t* dst = (SINGLE && out_pad) ? out + chunked_elem(tok, col0 + d, out_pad) : orow_p + d;
                    *(uint2*)dst = w.h[0];
                }
            }
        } else {
            const size_t prow = (size_t)split * total_rows + orow[rt];
            float* po = ws_o + prow * hd;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 16 + lg * 4;
                if (d < hd) *(floatx4_t*)(po + d) = o[rt][dt];
            }
            if (lg == 0) {
                ws_ml[prow * 2] = m[rt];
                ws_ml[prow * 2 + 1] = lt[rt];
            }
        }
    }
}

// --------------------------------------------------------------------------------------
// Prompts: a workgroup of four waves owns 128 or 64 query rows (RT tiles of 16 per wave) of
// one sequence and kv head and walks the keys a page (64 keys) at a time.  A page's keys and
// values - each one contiguous piece of the cache, already in the operands' order - are
// copied by all four waves straight into LDS (global_load_lds, 16 bytes per lane, no
// registers in between) while earlier pages are multiplied.
//
// The arithmetic is that of the kernel above, a page (64 keys) at a time.
// RT row tiles of 16 per wave: 2 (128 rows per workgroup) once such workgroups fill the slots
// of the chip (two per compute unit): an operand read from LDS then serves two matrix
// instructions; 1 (64 rows) for smaller grids, which need the workgroups more than the reuse
// (measured at head size 128, 8 kv heads: 1,536 tokens 37.8 us against 43.6, 2,048 tokens
// 58.7 against 54.7).
#define TL_WAVES 4

// FULL: the head size is exactly the one the tiles are laid out for (no edge tests).
// The running maximum of a row is only raised when a block's maximum exceeds it by more than
// TL_SLACK (in log2 units): probabilities then stay below 2^TL_SLACK, which float sums and the
// bfloat16 operand of the second product hold at full relative precision, and the output
// accumulators are rescaled rarely instead of nearly every block.
#define TL_SLACK 8.0f
template <int DS, bool FULL, int RT>
__global__ __launch_bounds__(256, 2) void attention_tiled_kernel(
        const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
        const bf16_t* __restrict__ v_pages, const int* __restrict__ q_start,
        const int* __restrict__ start_pos, const int* __restrict__ table, int table_stride,
        bf16_t* __restrict__ out, int H, int Hkv, int hd, float scale_log2, int window,
        int pair_from) {
    constexpr int DT = DS * 2;
    constexpr int TL_ROWS = TL_WAVES * RT * 16;
    constexpr int HDM = DS * 32;                          // head size the tiles are laid out for
    constexpr int KBYTES = 64 * HDM * 2, VBYTES = HDM * 64 * 2;   // a page's keys, its values
    constexpr int K_PER = KBYTES / 16 / 256, V_PER = VBYTES / 16 / 256;   // copies per thread
    // Two pages of keys and two of values, each an LDS object of its own: the compiler then
    // knows that a copy into one of them (global_load_lds) cannot change what the operand reads
    // take from the other, and does not make those reads wait for the copy.  With one array
    // indexed by the page's parity it put a wait for all copies in front of every page's
    // products, so that no copy overlapped the arithmetic of its own wave.
    __shared__ __attribute__((aligned(16))) char kb0[KBYTES];
    __shared__ __attribute__((aligned(16))) char kb1[KBYTES];
    __shared__ __attribute__((aligned(16))) char vb0[VBYTES];
    __shared__ __attribute__((aligned(16))) char vb1[VBYTES];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int seq = blockIdx.z;
    const int R = H / Hkv;
    const int q0 = q_start[seq];
    const int rows_total = (q_start[seq + 1] - q0) * R;
    // Later tiles see more keys.  Workgroups are handed out in the order of their linear
    // index; rank r in the order "most keys first" is tile gridDim.x - 1 - r / Hkv, head
    // r % Hkv.  Ranks are given out in descending work; if all workgroups fit the chip at
    // once (pair_from > 0: two per compute unit, index i + pair_from joining index i), the
    // joining half takes the light ranks lightest first, so that every compute unit holds
    // about the same number of keys.
    const int total = gridDim.x * gridDim.y;
    const int lin = blockIdx.x + gridDim.x * blockIdx.y;
    int rank = lin;
    if (pair_from > 0) {
        const int idx = (lin / (2 * pair_from)) * pair_from + lin % pair_from;
        rank = ((lin / pair_from) & 1) ? total - 1 - idx : idx;
    }
    const int g = rank % gridDim.y;
    const int wg_row0 = (gridDim.x - 1 - rank / gridDim.y) * TL_ROWS;
    if (wg_row0 >= rows_total) return;
    const int spos = start_pos[seq];
    const int* pages = table + (size_t)seq * table_stride;
    const int row0 = wg_row0 + wave * RT * 16;            // this wave's first row (may be beyond the end)

    Frag qf[RT][DS];
    int rpos[RT];
    size_t orow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int r = row0 + rt * 16 + li;
        const bool valid = r < rows_total;
        const int t = valid ? r / R : 0, hh = valid ? r - (r / R) * R : 0;
        rpos[rt] = valid ? spos + t : -1;
        orow[rt] = (size_t)(q0 + t) * H + g * R + hh;
        const bf16_t* qrow = q + orow[rt] * hd;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int d = ds * 32 + lg * 8;
            qf[rt][ds].u = (valid && (FULL || d < hd)) ? *(const uint4*)(qrow + d) : make_uint4(0, 0, 0, 0);
        }
    }
    // key range of the workgroup and of this wave
    const int wg_last = (wg_row0 + TL_ROWS - 1 < rows_total - 1) ? wg_row0 + TL_ROWS - 1 : rows_total - 1;
    const int wg_pmin = spos + wg_row0 / R, wg_pmax = spos + wg_last / R;
    const bool wave_has_rows = row0 < rows_total;
    const int w_last = (row0 + RT * 16 - 1 < rows_total - 1) ? row0 + RT * 16 - 1 : rows_total - 1;
    const int pmin = wave_has_rows ? spos + row0 / R : 0;
    const int pmax = wave_has_rows ? spos + w_last / R : -1;
    const int lo = (window > 0 && wg_pmin - window + 1 > 0) ? wg_pmin - window + 1 : 0;
    const int w_lo = (window > 0 && pmin - window + 1 > 0) ? pmin - window + 1 : 0;
    const int page_lo = lo >> 6, page_hi = wg_pmax >> 6;

    float m[RT], l[RT];
    floatx4_t o[RT][DT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[rt][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    // Copies.  A page's keys and its values lie in the cache in the order in which the operands
    // are read (common.h), so they are copied as they lie: thread t fills the 16-byte LDS slots
    // t + 256 i from the same places of the page (a wave's 64 slots are contiguous, as
    // global_load_lds writes them), and an operand read is 256 consecutive bytes per sixteen
    // lanes (keys) or 1 KB per wave (values): no two lanes of a pass share a bank.
    const int hdr = FULL ? HDM : hd;
    const int page_slots = 8 * hdr;                        // 16-byte slots of keys (of values) per page
    auto copy_keys = [&](int pg, char* kbuf) {
        const char* src = (const char*)(k_pages + cache_region(pages[pg], g, Hkv, hd)) + threadIdx.x * 16;
        char* dst = kbuf + wave * 1024;
#pragma unroll
        for (int i = 0; i < K_PER; ++i)
            if (FULL || (int)threadIdx.x + i * 256 < page_slots)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(src + i * 4096),
                    (__attribute__((address_space(3))) void*)(dst + i * 4096), 16, 0, 0);
    };
    auto copy_values = [&](int pg, char* vbuf) {
        const char* src = (const char*)(v_pages + cache_region(pages[pg], g, Hkv, hd)) + threadIdx.x * 16;
        char* dst = vbuf + wave * 1024;
#pragma unroll
        for (int i = 0; i < V_PER; ++i)
            if (FULL || (int)threadIdx.x + i * 256 < page_slots)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(src + i * 4096),
                    (__attribute__((address_space(3))) void*)(dst + i * 4096), 16, 0, 0);
    };
    // The copies of this thread have arrived.  Slots of the newest page that lie beyond the
    // newest key hold no data yet (whatever the cache held before): their values are set to
    // zero, by the thread that copied them, so that probability 0 times them is 0.  Value slot
    // s holds keys 32 (s / 64 % 2) + 8 (s / 16 % 4) .. + 7.
    auto copies_landed = [&](int v_pg, char* vt) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (v_pg > page_hi) return;
        const int keys_ok = wg_pmax - v_pg * 64;
        if (keys_ok >= 63) return;
#pragma unroll
        for (int i = 0; i < V_PER; ++i) {
            const int slot = threadIdx.x + i * 256;
            const int key_first = ((slot >> 6) & 1) * 32 + ((slot >> 4) & 3) * 8;
            if ((FULL || slot < page_slots) && key_first + 7 > keys_ok) {
                Frag f;
                f.u = *(const uint4*)(vt + slot * 16);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (key_first + e > keys_ok) f.e[e] = 0;
                *(uint4*)(vt + slot * 16) = f.u;
            }
        }
    };

    // operand reads: keys - chunk ds * 4 + lg of slot 16 t + li of block b, at
    // b * 64 hd + t * 256 + k_off[ds]; values - tile dt, block hb, at (2 dt + hb) * 1024 + lane * 16
    int k_off[DS];
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) k_off[ds] = (ds * 4 + lg) * 512 + li * 16;

    // The pages this wave has keys in (none: hi < lo).
    const int w_page_lo = (w_lo >> 6) > page_lo ? (w_lo >> 6) : page_lo;
    const int w_page_hi = wave_has_rows ? pmax >> 6 : -1;

    // A step works on two pages at once, so that matrix and vector instructions of one wave
    // have nothing to wait for in each other: the scores of page p + 1 (keys times queries) are
    // multiplied while the exponentials of page p are taken, and the second product of page p
    // (values times probabilities) while the row maxima of page p + 1 are.  The source gives
    // the order - one or two matrix instructions, then a few vector instructions that do not
    // need their result - and scheduling fences keep it.  `sc` holds the scores of page p,
    // masked, from the step before; m already covers them.
    floatx4_t sc[RT][4];
    auto step = [&](auto cur_tag, auto nxt_tag, int pg, const char* kt, const char* vt) {
        constexpr bool CUR = decltype(cur_tag)::value, NXT = decltype(nxt_tag)::value;
        floatx4_t s2[RT][4];
        Frag pf[RT][2];
        Frag kf[4][DS];
        Frag vf[DT][2];
        float neg_m[RT], sum[RT], p_e[RT][4];
        constexpr int KAHEAD = RT == 1 ? 4 : 2;            // key blocks requested ahead of their use
        constexpr int VAHEAD = RT == 1 ? DT : (DT + 1) / 2;
        auto read_keys = [&](int kt16) {
#pragma unroll
            for (int ds = 0; ds < DS; ++ds)
                kf[kt16][ds].u = (FULL || ds * 32 + lg * 8 < hd)
                                     ? *(const uint4*)(kt + (kt16 >> 1) * 64 * hdr + (kt16 & 1) * 256 + k_off[ds])
                                     : make_uint4(0, 0, 0, 0);
        };
        auto read_values = [&](int dt) {
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) vf[dt][hb].u = *(const uint4*)(vt + (dt * 2 + hb) * 1024 + lane * 16);
        };
        if (NXT) {
#pragma unroll
            for (int kt16 = 0; kt16 < KAHEAD; ++kt16) read_keys(kt16);
        }
        if (CUR) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                neg_m[rt] = (m[rt] == -INFINITY) ? 0.f : -m[rt];
                sum[rt] = 0.f;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // scores of page pg + 1 | exponentials of page pg
#pragma unroll
        for (int kt16 = 0; kt16 < 4; ++kt16) {
            if (NXT && kt16 + KAHEAD < 4) read_keys(kt16 + KAHEAD);
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) {
                if (NXT) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        s2[rt][kt16] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            kf[kt16][ds].v, qf[rt][ds].v, ds == 0 ? floatx4_t{0.f, 0.f, 0.f, 0.f} : s2[rt][kt16], 0, 0, 0);
                }
                if (CUR) {
                    // the four scores of key block kt16, one per matrix instruction (a head
                    // size of 64 has two per block: two scores each)
                    constexpr int PER = 4 / DS;
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                        for (int j = ds * PER; j < (ds + 1) * PER; ++j) {
                            p_e[rt][j] = __builtin_amdgcn_exp2f(fmaf(sc[rt][kt16][j], scale_log2, neg_m[rt]));
                            sum[rt] += p_e[rt][j];
                            // computed here, between the matrix instructions, not where the
                            // second product uses it (the compiler would sink it there)
                            asm volatile("" : "+v"(p_e[rt][j]), "+v"(sum[rt]));
                        }
                        if (ds == DS - 1) {
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                pf[rt][kt16 >> 1].e[(kt16 & 1) * 4 + j] = float_to_bf16(p_e[rt][j]);
                            if (kt16 & 1) asm volatile("" : "+v"(pf[rt][kt16 >> 1].u.z), "+v"(pf[rt][kt16 >> 1].u.w));
                            else asm volatile("" : "+v"(pf[rt][kt16 >> 1].u.x), "+v"(pf[rt][kt16 >> 1].u.y));
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (CUR) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) l[rt] += sum[rt];
#pragma unroll
            for (int dt = 0; dt < VAHEAD; ++dt) read_values(dt);
        }
        __builtin_amdgcn_sched_barrier(0);
        float mx[RT];
        if (NXT) {
            const int p2 = pg + 1;
            const bool masked = p2 * 64 + 63 > pmin || (window > 0 && p2 * 64 < pmax - window + 1);
            if (masked) {
                const int key0 = p2 * 64 + lg * 8;         // this lane's keys: key0 .. +7, key0 + 32 .. +39
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const int first = (window > 0) ? rpos[rt] - window + 1 : 0;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = key0 + (e >> 3) * 32 + (e & 7);
                        if (!(key <= rpos[rt] && key >= first)) s2[rt][e >> 2][e & 3] = -INFINITY;
                    }
                }
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) mx[rt] = -INFINITY;
        }
        __builtin_amdgcn_sched_barrier(0);
        // second product of page pg | row maxima of page pg + 1
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (CUR) {
                if (dt + VAHEAD < DT) read_values(dt + VAHEAD);
                // every tile of dims is multiplied, also those beyond a smaller head (what LDS
                // holds there goes into accumulators that are never stored)
#pragma unroll
                for (int hb = 0; hb < 2; ++hb) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt][hb].v, pf[rt][hb].v, o[rt][dt], 0, 0, 0);
                }
            }
            if (NXT) {
                // DT is 4 or 8: the sixteen scores of a row tile in DT steps
                constexpr int PER = 16 / DT;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                    for (int e = dt * PER; e < (dt + 1) * PER; ++e) mx[rt] = fmaxf(mx[rt], s2[rt][e >> 2][e & 3]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (NXT) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float top = max_over_lane_groups(mx[rt]) * scale_log2;   // scale > 0: the order is kept
                if (__builtin_amdgcn_ballot_w64(top > m[rt] + TL_SLACK) != 0) {
                    // some row's maximum moved far: raise every row's reference and rescale
                    const float m_new = fmaxf(m[rt], top);
                    const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m[rt] - m_new);
                    l[rt] *= alpha;
                    m[rt] = m_new;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) o[rt][dt] *= alpha;
                }
#pragma unroll
                for (int kt16 = 0; kt16 < 4; ++kt16) sc[rt][kt16] = s2[rt][kt16];
            }
        }
    };
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;

    // Step pg reads the keys of page pg + 1 and the values of page pg, while the copies of the
    // keys of page pg + 2 and the values of page pg + 1 are on their way into the buffers that
    // the step before has read last.  The first step (pg = page_lo - 1) has no page of its own.
    copy_keys(page_lo, kb0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#define TL_STEP(PG, KNEXT, KFREE, VCUR, VFREE)                                                   \
    {                                                                                            \
        if ((PG) + 2 <= page_hi) copy_keys((PG) + 2, KFREE);                                     \
        if ((PG) + 1 <= page_hi) copy_values((PG) + 1, VFREE);                                   \
        const bool cur = (PG) >= w_page_lo && (PG) <= w_page_hi;                                 \
        const bool nxt = (PG) + 1 >= w_page_lo && (PG) + 1 <= w_page_hi;                         \
        if (cur && nxt) step(Yes{}, Yes{}, PG, KNEXT, VCUR);                                     \
        else if (cur) step(Yes{}, No{}, PG, KNEXT, VCUR);                                        \
        else if (nxt) step(No{}, Yes{}, PG, KNEXT, VCUR);                                        \
        copies_landed((PG) + 1, VFREE);                                                          \
        __syncthreads();                                                                         \
    }
    for (int pg = page_lo - 1; pg <= page_hi; pg += 2) {
        TL_STEP(pg, kb0, kb1, vb1, vb0)
        if (pg + 1 <= page_hi) TL_STEP(pg + 1, kb1, kb0, vb0, vb1)
    }
#undef TL_STEP

#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const float lt = sum_over_lane_groups(l[rt]);
        if (rpos[rt] < 0) continue;
        const float inv = 1.f / lt;
        bf16_t* orow_p = out + orow[rt] * hd;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int d = dt * 16 + lg * 4;
            if (d < hd) {
                Frag w;
#pragma unroll
                for (int j = 0; j < 4; ++j) w.e[j] = float_to_bf16(o[rt][dt][j] * inv);
                *(uint2*)(orow_p + d) = w.h[0];
            }
        }
    }
}

template <int DS, bool FULL, int RT>
static void launch_attention_tiled_rt(dim3 grid, int slots, hipStream_t stream, const bf16_t* q,
                                      const bf16_t* k, const bf16_t* v, const int* q_start,
                                      const int* start_pos, const int* table, int table_stride,
                                      bf16_t* out, int H, int Hkv, int hd, float sl2, int window) {
    constexpr int HDM = DS * 32;
    const int total = (int)(grid.x * grid.y);
    const int pair_from = (grid.z == 1 && total > 1 && total <= slots && total % 2 == 0) ? total / 2 : 0;
    attention_tiled_kernel<DS, FULL, RT><<<grid, 256, 0, stream>>>(
        q, k, v, q_start, start_pos, table, table_stride, out, H, Hkv, hd, sl2, window, pair_from);
}

template <int DS, bool FULL>
static void launch_attention_tiled(int max_rows, int n_seqs, int row_tiles, hipStream_t stream, const bf16_t* q,
                                   const bf16_t* k, const bf16_t* v, const int* q_start,
                                   const int* start_pos, const int* table, int table_stride,
                                   bf16_t* out, int H, int Hkv, int hd, float sl2, int window) {
    static int slots = 0;                                  // workgroups the chip holds at once
    if (slots == 0) {
        int dev = 0, cus = 0;
        hipGetDevice(&dev);
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        slots = 2 * (cus > 0 ? cus : 1);
    }
    const int tiles128 = (max_rows + 127) / 128;
    if (row_tiles == 0) row_tiles = ((long)tiles128 * Hkv * n_seqs < slots) ? 1 : 2;
    if (row_tiles == 1)
        launch_attention_tiled_rt<DS, FULL, 1>(dim3((max_rows + 63) / 64, Hkv, n_seqs), slots, stream, q, k, v,
                                               q_start, start_pos, table, table_stride, out, H, Hkv, hd, sl2, window);
    else
        launch_attention_tiled_rt<DS, FULL, 2>(dim3(tiles128, Hkv, n_seqs), slots, stream, q, k, v, q_start,
                                               start_pos, table, table_stride, out, H, Hkv, hd, sl2, window);
}

// Prompts of many rows: max_rows = most (token, head of a group) rows any sequence has per kv
// head; row_tiles = 16-row tiles per wave, 1 or 2, or 0 to let the size of the grid choose.
extern "C" int gfa_attention_tiled_bf16(const void* q, const void* k_pages, const void* v_pages,
                                        const int* q_start, const int* start_pos, const int* table,
                                        int table_stride, void* out, int n_tokens, int n_seqs, int H,
                                        int Hkv, int hd, float scale, int window, int max_rows,
                                        int row_tiles, hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (hd % 16 != 0 || hd > 128 || H % Hkv != 0 || max_rows < 1 || row_tiles < 0 || row_tiles > 2 ||
        !(scale > 0.f))                                   // the kernels take maxima before scaling
        return (int)hipErrorInvalidValue;
    const float sl2 = scale * LOG2E;
    const bf16_t* qp = (const bf16_t*)q;
    const bf16_t* kp = (const bf16_t*)k_pages;
    const bf16_t* vp = (const bf16_t*)v_pages;
    bf16_t* op = (bf16_t*)out;
    if (hd == 64) launch_attention_tiled<2, true>(max_rows, n_seqs, row_tiles, stream, qp, kp, vp, q_start, start_pos, table, table_stride, op, H, Hkv, hd, sl2, window);
    else if (hd < 64) launch_attention_tiled<2, false>(max_rows, n_seqs, row_tiles, stream, qp, kp, vp, q_start, start_pos, table, table_stride, op, H, Hkv, hd, sl2, window);
    else if (hd == 128) launch_attention_tiled<4, true>(max_rows, n_seqs, row_tiles, stream, qp, kp, vp, q_start, start_pos, table, table_stride, op, H, Hkv, hd, sl2, window);
    else launch_attention_tiled<4, false>(max_rows, n_seqs, row_tiles, stream, qp, kp, vp, q_start, start_pos, table, table_stride, op, H, Hkv, hd, sl2, window);
    return GFA_LAUNCH_RESULT();
}

// out[row, :] = sum_s w_s o_s / sum_s w_s l_s with w_s = 2^(m_s - max m), splits in order.
// One wave per row.  Lane s holds split s's maximum and sum (at most 64 splits); the loads
// of the partial results do not depend on each other, so a batch of them is in flight at
// once instead of one round trip per split.
__global__ __launch_bounds__(64) void attention_combine_kernel(const float* __restrict__ ws_o,
                                                               const float* __restrict__ ws_ml,
                                                               bf16_t* __restrict__ out, int hd,
                                                               int n_splits, int total_rows, int H,
                                                               int out_pad) {
    const int row = blockIdx.x, lane = threadIdx.x;      // row = token * H + head
    float ms = -INFINITY, ls = 0.f;
    if (lane < n_splits) {
        const float2 ml = *(const float2*)(ws_ml + ((size_t)lane * total_rows + row) * 2);
        ms = ml.x;
        ls = ml.y;
    }
    const float mmax = wave_max(ms);
    const float wgt = (ms == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ms - mmax);   // a split without keys: 0
    float den = 0.f;
    for (int sp = 0; sp < n_splits; ++sp) den += __shfl(wgt * ls, sp, 64);
    const float inv = 1.f / den;
    // every lane runs the loop (the weights come from other lanes by shuffles); a lane whose
    // two dims lie beyond the head neither loads nor stores
    for (int d0 = 0; d0 < hd; d0 += 128) {
        const int d = d0 + lane * 2;
        const bool mine = d < hd;
        const float* src = ws_o + (size_t)row * hd + (mine ? d : 0);
        const size_t stride = (size_t)total_rows * hd;
        float a0 = 0.f, a1 = 0.f;
        int sp = 0;
        for (; sp + 8 <= n_splits; sp += 8) {
            float2 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = *(const float2*)(src + (sp + j) * stride);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float wj = __shfl(wgt, sp + j, 64);
                a0 += wj * v[j].x;
                a1 += wj * v[j].y;
            }
        }
        for (; sp < n_splits; ++sp) {
            const float2 v = *(const float2*)(src + sp * stride);
            const float wj = __shfl(wgt, sp, 64);
            a0 += wj * v.x;
            a1 += wj * v.y;
        }
        if (mine) {
            // out_pad: left chunked (common.h) for the product that reads it next
            bf16_t* dst = out_pad ? out + chunked_elem(row / H, (row % H) * hd + d, out_pad)
                                  : out + (size_t)row * hd + d;
            dst[0] = float_to_bf16(a0 * inv);
            dst[1] = float_to_bf16(a1 * inv);
        }
    }
}

template <int DS>
static void launch_attention(int rt, int nw, dim3 grid, hipStream_t stream, const bf16_t* q,
                             const bf16_t* k, const bf16_t* v, const int* q_start,
                             const int* start_pos, const int* table, int table_stride, bf16_t* out,
                             float* ws_o, float* ws_ml, int H, int Hkv, int hd, float sl2, int window,
                             int n_splits, int total_rows, bool single, int out_pad) {
    const size_t shmem = nw > 1 ? (size_t)(nw - 1) * rt * (16 * 2 * sizeof(float) + DS * 2 * 64 * sizeof(floatx4_t)) : 0;
    if (rt == 1 && single)
        attention_mfma_kernel<DS, 1, false, true><<<dim3(n_splits, grid.y, grid.z / n_splits), 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, out_pad, SlicedRowsIn{});
    else if (rt == 1)
        attention_mfma_kernel<DS, 1, false><<<grid, 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, 0, SlicedRowsIn{});
    else if (rt == 2)
        attention_mfma_kernel<DS, 2, (DS <= 4)><<<grid, 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, 0, SlicedRowsIn{});
    else if (DS <= 4)
        attention_mfma_kernel<(DS <= 4 ? DS : 4), 4, false><<<grid, 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, 0, SlicedRowsIn{});
}

// q, out [n_tokens, H, hd]; the sequences' token runs are given by q_start [n_seqs + 1] and
// their first positions by start_pos [n_seqs].  rt (1, 2 or 4) 16-row tiles per wave;
// n_waves (1..4; up to 8 with rt 1) waves per workgroup share the key blocks of their rows;
// max_tiles = most waves any sequence needs per kv head.  With n_splits > 1, ws_o
// [n_splits, n_tokens * H, hd] and ws_ml [n_splits, n_tokens * H, 2] hold the partials.
// one_token_each: the caller vouches that q_start is 0, 1, 2, ... (every sequence one token).
// out_chunked (with one_token_each, up to 64 tokens): out is left as chunked rows [n_tokens,
// H * hd] (common.h: chunked_elem) for the few-row product that reads it.
extern "C" int gfa_attention_bf16(const void* q, const void* k_pages, const void* v_pages,
                                  const int* q_start, const int* start_pos, const int* table,
                                  int table_stride, void* out, float* ws_o, float* ws_ml,
                                  int n_tokens, int n_seqs, int H, int Hkv, int hd, float scale,
                                  int window, int rt, int n_waves, int max_tiles, int n_splits,
                                  int one_token_each, int out_chunked, hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (one_token_each && n_tokens != n_seqs) return (int)hipErrorInvalidValue;
    if ((long)table_stride * 2 * (n_splits + 1) >= (1L << 31)) return (int)hipErrorInvalidValue;
    const bool single = one_token_each && rt == 1 && max_tiles == 1 && H / Hkv <= 16;
    // out_chunked: up to 64 tokens, one per sequence, (H * hd) % 8 == 0 (it is: hd % 16 == 0)
    if (out_chunked && (!single || n_tokens > 64)) return (int)hipErrorInvalidValue;
    const int out_pad = !out_chunked ? 0 : n_tokens <= 4 ? 4 : n_tokens <= 8 ? 8 : n_tokens <= 16 ? 16
                                         : n_tokens <= 32 ? 32 : 64;
    if (hd % 16 != 0 || hd > 256 || H % Hkv != 0 || n_splits < 1 || n_splits > 64 || max_tiles < 1 ||
        !(scale > 0.f) ||                                 // the kernels take maxima before scaling
        (rt != 1 && rt != 2 && rt != 4) || (rt == 4 && hd > 128) ||
        (n_splits > 1 && (!ws_o || !ws_ml)) || n_waves < 1 || n_waves > (rt == 1 ? 8 : 4) ||
        (size_t)(n_waves - 1) * rt * (128 + (hd <= 64 ? 2 : hd <= 128 ? 4 : 8) * 2 * 1024) > 65536)
        return (int)hipErrorInvalidValue;
    const dim3 grid(max_tiles, Hkv, n_seqs * n_splits);
    const float sl2 = scale * LOG2E;
    const int total_rows = n_tokens * H;
    const bf16_t* qp = (const bf16_t*)q;
    const bf16_t* kp = (const bf16_t*)k_pages;
    const bf16_t* vp = (const bf16_t*)v_pages;
    if (hd <= 64)
        launch_attention<2>(rt, n_waves, grid, stream, qp, kp, vp, q_start, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, single, out_pad);
    else if (hd <= 128)
        launch_attention<4>(rt, n_waves, grid, stream, qp, kp, vp, q_start, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, single, out_pad);
    else
        launch_attention<8>(rt, n_waves, grid, stream, qp, kp, vp, q_start, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows, single, out_pad);
    if (n_splits > 1)
        attention_combine_kernel<<<total_rows, 64, 0, stream>>>(ws_o, ws_ml, (bf16_t*)out, hd, n_splits, total_rows, H, out_pad);
    return GFA_LAUNCH_RESULT();
}

// One token per sequence whose q, k and v rows are still the float partial sums part
// [S, n_seqs, (H + 2 Hkv) * hd] of a sliced product: the slices are added, queries and key
// rotated (interleaved pairs, rot a multiple of 4, frequencies freqs [rot / 2]) and attended in
// one kernel, and the new keys and values written to the cache (k_pages / v_pages; a run that
// reads another run's cache gives write_cache = 0).  out [n_seqs, H, hd]; start_pos [n_seqs] is
// each token's position; head sizes up to 128, at most sixteen query heads per kv head.
extern "C" int gfa_attention_sliced_bf16(const float* part, int S, const float* freqs, int rot,
                                         void* k_pages, void* v_pages, int write_cache,
                                         const int* start_pos, const int* table, int table_stride,
                                         void* out, float* ws_o, float* ws_ml, int n_seqs, int H,
                                         int Hkv, int hd, float scale, int window, int n_waves,
                                         int n_splits, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if ((long)table_stride * 2 * (n_splits + 1) >= (1L << 31)) return (int)hipErrorInvalidValue;
    if (!part || S < 1 || hd % 16 != 0 || hd > 128 || Hkv < 1 || H % Hkv != 0 || H / Hkv > 16 ||
        rot < 0 || rot % 4 != 0 || rot > hd || rot > SL_MAX_ROT || (rot > 0 && !freqs) ||
        (H / Hkv + 2) * hd > SL_MAX_ELEMS || n_splits < 1 || n_splits > 64 || !(scale > 0.f) ||
        (n_splits > 1 && (!ws_o || !ws_ml)) || n_waves < 1 || n_waves > 8 ||
        (size_t)(n_waves - 1) * (128 + (hd <= 64 ? 2 : 4) * 2 * 1024) > 65536)
        return (int)hipErrorInvalidValue;
    const int width = (H + 2 * Hkv) * hd;
    const SlicedRowsIn sl = {part, S, (size_t)n_seqs * width, width, freqs, rot,
                             write_cache ? (bf16_t*)k_pages : nullptr,
                             write_cache ? (bf16_t*)v_pages : nullptr};
    const float sl2 = scale * LOG2E;
    const int total_rows = n_seqs * H;
    const dim3 grid(n_splits, Hkv, n_seqs);
    const bf16_t* kp = (const bf16_t*)k_pages;
    const bf16_t* vp = (const bf16_t*)v_pages;
    if (hd <= 64) {
        const size_t shmem = n_waves > 1 ? (size_t)(n_waves - 1) * (16 * 2 * sizeof(float) + 2 * 2 * 64 * sizeof(floatx4_t)) : 0;
        attention_mfma_kernel<2, 1, false, true, true><<<grid, 64 * n_waves, shmem, stream>>>(
            nullptr, kp, vp, nullptr, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv,
            hd, sl2, window, n_splits, total_rows, 0, sl);
    } else {
        const size_t shmem = n_waves > 1 ? (size_t)(n_waves - 1) * (16 * 2 * sizeof(float) + 4 * 2 * 64 * sizeof(floatx4_t)) : 0;
        attention_mfma_kernel<4, 1, false, true, true><<<grid, 64 * n_waves, shmem, stream>>>(
            nullptr, kp, vp, nullptr, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv,
            hd, sl2, window, n_splits, total_rows, 0, sl);
    }
    if (n_splits > 1)
        attention_combine_kernel<<<total_rows, 64, 0, stream>>>(ws_o, ws_ml, (bf16_t*)out, hd, n_splits, total_rows, H, 0);
    return GFA_LAUNCH_RESULT();
}
