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

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

union Frag {
    uint4 u;
    uint2 h[2];
    bf16_t e[8];
    bf16x8_t v;
};

#define LOG2E 1.4426950408889634f

template <int DS, int RT, bool PREFETCH>
__global__ __launch_bounds__(256) void attention_mfma_kernel(
        const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
        const bf16_t* __restrict__ v_pages, const int* __restrict__ q_start,
        const int* __restrict__ start_pos, const int* __restrict__ table, int table_stride,
        bf16_t* __restrict__ out, float* __restrict__ ws_o, float* __restrict__ ws_ml, int H,
        int Hkv, int hd, float scale_log2, int window, int n_splits, int total_rows) {
    constexpr int DT = DS * 2;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int g = blockIdx.y;
    const int seq = blockIdx.z / n_splits, split = blockIdx.z - seq * n_splits;
    const int R = H / Hkv;
    const int q0 = q_start[seq];
    const int rows_total = (q_start[seq + 1] - q0) * R;
    const int row0 = blockIdx.x * 16 * RT;
    if (row0 >= rows_total) return;                      // the whole workgroup leaves
    const int spos = start_pos[seq];
    const int* pages = table + (size_t)seq * table_stride;

    Frag qf[RT][DS];
    int rpos[RT];             // position of this lane's row in tile rt, -1 if there is none
    size_t orow[RT];          // (token, head) index of that row in q / out
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
            qf[rt][ds].u = (valid && d < hd) ? *(const uint4*)(qrow + d) : make_uint4(0, 0, 0, 0);
        }
    }
    const int last_row = (row0 + 16 * RT - 1 < rows_total - 1) ? row0 + 16 * RT - 1 : rows_total - 1;
    const int pmin = spos + row0 / R, pmax = spos + last_row / R;
    const int lo = (window > 0 && pmin - window + 1 > 0) ? pmin - window + 1 : 0;
    const int kb_lo = lo >> 5, nkb = (pmax >> 5) - kb_lo + 1;
    const int kb_begin = kb_lo + (int)((long)split * nkb / n_splits);
    const int kb_end = kb_lo + (int)((long)(split + 1) * nkb / n_splits);

    float m[RT], l[RT];
    floatx4_t o[RT][DT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[rt][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    // keys: tile kt, row kt * 16 + li of the block, dims ds * 32 + lg * 8 .. +7
    // values: dims dt * 16 + li, keys (tile 0 | tile 1) 4 lg .. +3 of the block
    auto load_block = [&](int kb, Frag (&kf)[2][DS], Frag (&vf)[DT]) {
        const int page = pages[kb >> 1];
        const int in_page = (kb & 1) * 32;
        const bf16_t* kbase = k_pages + page_row(page, g, in_page, Hkv, hd);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) {
                const int d = ds * 32 + lg * 8;
                kf[kt][ds].u = (d < hd) ? *(const uint4*)(kbase + (size_t)(kt * 16 + li) * hd + d)
                                        : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int d = dt * 16 + li;
            if (d < hd) {
                const bf16_t* vrow = v_pages + value_elem(page, g, d, in_page + lg * 4, Hkv, hd);
                vf[dt].h[0] = *(const uint2*)vrow;
                vf[dt].h[1] = *(const uint2*)(vrow + 16);
            } else {
                vf[dt].u = make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto compute_block = [&](int kb, Frag (&kf)[2][DS], Frag (&vf)[DT]) {
        const int key0 = kb * 32 + lg * 4;
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
                    if (key0 + (e >> 2) * 16 + (e & 3) > pmax) vf[dt].e[e] = 0;
        }
        // blocks wholly below every row's position (and inside every window) need no mask
        const bool masked = kb * 32 + 31 > pmin || (window > 0 && kb * 32 < pmax - window + 1);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            float sv[8];
            float mx = -INFINITY;
            if (masked) {
                const int first = (window > 0) ? rpos[rt] - window + 1 : 0;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = key0 + (e >> 2) * 16 + (e & 3);
                    const float v = s[rt][e >> 2][e & 3] * scale_log2;
                    sv[e] = (key <= rpos[rt] && key >= first) ? v : -INFINITY;
                    mx = fmaxf(mx, sv[e]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    sv[e] = s[rt][e >> 2][e & 3] * scale_log2;
                    mx = fmaxf(mx, sv[e]);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m[rt], mx);
            // a row without any key so far keeps m = -inf: exp2(-inf - -inf) must not be formed
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m[rt] - m_safe);
            Frag pf;
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = __builtin_amdgcn_exp2f(sv[e] - m_safe);      // 2^-inf = 0
                sum += p;
                pf.e[e] = float_to_bf16(p);
            }
            l[rt] = l[rt] * alpha + sum;
            m[rt] = m_new;
            // the running maximum rarely moves after the first blocks: skip the rescale then
            const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                if (dt * 16 < hd) {
                    if (rescale) o[rt][dt] *= alpha;
                    o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf.v, o[rt][dt], 0, 0, 0);
                }
            }
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
        lt[rt] = l[rt] + __shfl_xor(l[rt], 16, 64);
        lt[rt] += __shfl_xor(lt[rt], 32, 64);
    }
    if (nw > 1) {                 // the waves' partial results meet in LDS, added in wave order
        float* sm_ml = (float*)smem;                                  // [nw][RT][16][2]
        floatx4_t* sm_o = (floatx4_t*)(smem + (size_t)nw * RT * 16 * 2 * sizeof(float));
        if (wave > 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if (lg == 0) {
                    sm_ml[((wave * RT + rt) * 16 + li) * 2] = m[rt];
                    sm_ml[((wave * RT + rt) * 16 + li) * 2 + 1] = lt[rt];
                }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) sm_o[((wave * RT + rt) * DT + dt) * 64 + lane] = o[rt][dt];
            }
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < nw; ++w)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float mw = sm_ml[((w * RT + rt) * 16 + li) * 2];
                if (mw == -INFINITY) continue;
                const float lw = sm_ml[((w * RT + rt) * 16 + li) * 2 + 1];
                const float m_new = fmaxf(m[rt], mw);
                const float a = __builtin_amdgcn_exp2f(m[rt] - m_new);     // 0 if this wave saw no key
                const float b = __builtin_amdgcn_exp2f(mw - m_new);
                lt[rt] = lt[rt] * a + lw * b;
                m[rt] = m_new;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    o[rt][dt] = o[rt][dt] * a + sm_o[((w * RT + rt) * DT + dt) * 64 + lane] * b;
            }
    }

#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rpos[rt] < 0) continue;
        if (n_splits == 1) {
            const float inv = 1.f / lt[rt];
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

// out[row, :] = sum_s w_s o_s / sum_s w_s l_s with w_s = 2^(m_s - max m), splits in order.
__global__ void attention_combine_kernel(const float* __restrict__ ws_o,
                                         const float* __restrict__ ws_ml, bf16_t* __restrict__ out,
                                         int hd, int n_splits, int total_rows) {
    const int row = blockIdx.x;
    float mmax = -INFINITY;
    for (int s = 0; s < n_splits; ++s) mmax = fmaxf(mmax, ws_ml[((size_t)s * total_rows + row) * 2]);
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float acc = 0.f, den = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const size_t prow = (size_t)s * total_rows + row;
            const float ms = ws_ml[prow * 2];
            if (ms == -INFINITY) continue;            // a split without keys
            const float wgt = __builtin_amdgcn_exp2f(ms - mmax);
            den += wgt * ws_ml[prow * 2 + 1];
            acc += wgt * ws_o[prow * hd + d];
        }
        out[(size_t)row * hd + d] = float_to_bf16(acc / den);
    }
}

template <int DS>
static void launch_attention(int rt, int nw, dim3 grid, hipStream_t stream, const bf16_t* q,
                             const bf16_t* k, const bf16_t* v, const int* q_start,
                             const int* start_pos, const int* table, int table_stride, bf16_t* out,
                             float* ws_o, float* ws_ml, int H, int Hkv, int hd, float sl2, int window,
                             int n_splits, int total_rows) {
    const size_t shmem = nw > 1 ? (size_t)nw * rt * (16 * 2 * sizeof(float) + DS * 2 * 64 * sizeof(floatx4_t)) : 0;
    if (rt == 1)
        attention_mfma_kernel<DS, 1, false><<<grid, 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows);
    else if (rt == 2)
        attention_mfma_kernel<DS, 2, (DS <= 4)><<<grid, 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows);
    else if (DS <= 4)
        attention_mfma_kernel<(DS <= 4 ? DS : 4), 4, false><<<grid, 64 * nw, shmem, stream>>>(q, k, v, q_start, start_pos, table, table_stride, out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows);
}

// q, out [n_tokens, H, hd]; the sequences' token runs are given by q_start [n_seqs + 1] and
// their first positions by start_pos [n_seqs].  rt (1, 2 or 4) 16-row tiles per wave;
// n_waves (1..4) waves per workgroup share the key blocks of their rows;
// max_tiles = most waves any sequence needs per kv head.  With n_splits > 1, ws_o
// [n_splits, n_tokens * H, hd] and ws_ml [n_splits, n_tokens * H, 2] hold the partials.
extern "C" int gfa_attention_bf16(const void* q, const void* k_pages, const void* v_pages,
                                  const int* q_start, const int* start_pos, const int* table,
                                  int table_stride, void* out, float* ws_o, float* ws_ml,
                                  int n_tokens, int n_seqs, int H, int Hkv, int hd, float scale,
                                  int window, int rt, int n_waves, int max_tiles, int n_splits,
                                  hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (hd % 16 != 0 || hd > 256 || H % Hkv != 0 || n_splits < 1 || max_tiles < 1 ||
        (rt != 1 && rt != 2 && rt != 4) || (rt == 4 && hd > 128) ||
        (n_splits > 1 && (!ws_o || !ws_ml)) || n_waves < 1 || n_waves > 4 ||
        (size_t)n_waves * rt * (128 + (hd <= 64 ? 2 : hd <= 128 ? 4 : 8) * 2 * 1024) > 65536)
        return (int)hipErrorInvalidValue;
    const dim3 grid(max_tiles, Hkv, n_seqs * n_splits);
    const float sl2 = scale * LOG2E;
    const int total_rows = n_tokens * H;
    const bf16_t* qp = (const bf16_t*)q;
    const bf16_t* kp = (const bf16_t*)k_pages;
    const bf16_t* vp = (const bf16_t*)v_pages;
    if (hd <= 64)
        launch_attention<2>(rt, n_waves, grid, stream, qp, kp, vp, q_start, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows);
    else if (hd <= 128)
        launch_attention<4>(rt, n_waves, grid, stream, qp, kp, vp, q_start, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows);
    else
        launch_attention<8>(rt, n_waves, grid, stream, qp, kp, vp, q_start, start_pos, table, table_stride, (bf16_t*)out, ws_o, ws_ml, H, Hkv, hd, sl2, window, n_splits, total_rows);
    if (n_splits > 1)
        attention_combine_kernel<<<total_rows, 64, 0, stream>>>(ws_o, ws_ml, (bf16_t*)out, hd, n_splits, total_rows);
    return GFA_LAUNCH_RESULT();
}
