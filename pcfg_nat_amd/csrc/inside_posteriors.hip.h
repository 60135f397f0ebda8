// Posteriors of long graphs from the tables the sweeps leave: emission cells element-wise, rule posteriors as a
// contraction over the target positions on the matrix cores (fp32 MFMA) with a term-by-term path where the range fails.
// Part of inside.hip (one translation unit: the kernels share helpers and the anonymous namespace).
#pragma once
#include "inside_common.hip.h"

namespace pcfgnat {
namespace {

// Emission posteriors (element-wise) from BETA, F0, F1: the epilogue of the register-resident backward, for the long
// graphs a kernel of its own or the work of the rule posterior launch's spare workgroups.
struct MatchGradArgs {
    const float *match_all;
    float *mgrad;  // null: the caller has a launch of its own for them
};

// The cells first, first + stride, ... of sentence b (cell i = node i / T, position i % T), NB of them at a time with
// every load of the batch issued ahead of its arithmetic: addresses of terms a cell does not have fall back to offset 0.
template <int NB>
__device__ __forceinline__ void match_grad_cells(const int b, const int first, const int stride, const float *__restrict__ grad_out,
                                                 const float *__restrict__ S, const float *__restrict__ aux_c,
                                                 const float *__restrict__ match_all, const int64_t *__restrict__ out_len,
                                                 const int64_t *__restrict__ tgt_len, float *__restrict__ mgrad, int L, int T, int Mc,
                                                 Seed seed, int use_corr) {
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *Sb = S + (size_t)b * Mc * (T + 2);
    const float *mt = match_all + (size_t)b * L * T;
    float *mg = mgrad + (size_t)b * L * T;
    const float ll = Sb[0];
    const int cells = L * T;
    if (!(lengths_ok(m, n, L, T) && (ll == ll) && (fabsf(ll) != __builtin_huge_valf()))) {
        for (int i = first; i < cells; i += stride) mg[i] = 0.f;
        return;
    }
    const int mc = m / 2;
    AuxViewStream av(const_cast<float *>(aux_c), b, Mc, T);
    const float g = seed_weight(grad_out, b, n, seed);
    // corrections of the columns (see pipeline_finish_kernel): on the forward's offsets they are 0 and -D_t
    const float *corr = ExchangeView(const_cast<float *>(aux_c), b, Mc, T).corr;
    const float *shift1 = use_corr ? corr + corr_len(T) : av.D;  // the second correction, or (negated) the forward's shift
    for (int i0 = first; i0 < cells; i0 += NB * stride) {
        float bs[NB], bp[NB], mx[NB], mo[NB], f0[NB], f1[NB], c0[NB], c1[NB];
        bool t_main[NB], t_prev[NB], t_last[NB], t_leaf[NB];
#pragma unroll
        for (int u = 0; u < NB; u++) {
            const int i = i0 + u * stride;
            const bool in = i < cells;
            const int x = in ? i / T : 0, s = in ? i - x * T : 0, a_id = x >> 1;
            const bool cell = in && x >= 1 && x < m && s < n, odd = (x & 1) != 0;
            t_main[u] = cell && odd && s + 1 <= n - 1;
            t_prev[u] = cell && odd && s >= 1 && s + 1 <= n - 1 && a_id >= 1;
            t_last[u] = cell && odd && a_id == mc - 1 && s == n - 1;
            t_leaf[u] = cell && !odd && a_id >= 1 && a_id < mc && s + 2 <= n - 1;
            const bool any = t_main[u] || t_prev[u] || t_last[u] || t_leaf[u];
            const size_t row = any ? (size_t)a_id * (T + 2) : 0;
            const int sa = any ? s : 0;
            bs[u] = av.BETA[row + sa];
            bp[u] = av.BETA[t_prev[u] ? row + sa - 1 : 0];
            mx[u] = mt[any ? (size_t)x * T + sa : 0];
            mo[u] = mt[t_prev[u] ? (size_t)(x - 1) * T + sa - 1 : (t_leaf[u] ? (size_t)(x + 1) * T + sa + 1 : 0)];
            f0[u] = av.F0[t_main[u] ? row + sa + 1 : 0];
            f1[u] = av.F1[t_prev[u] ? row + sa + 1 : (t_leaf[u] ? row + sa + 2 : 0)];
            c0[u] = use_corr ? corr[sa] : 0.f;
            c1[u] = shift1[t_leaf[u] ? sa + 1 : sa];
        }
#pragma unroll
        for (int u = 0; u < NB; u++) {
            const int i = i0 + u * stride;
            if (i >= cells) break;
            const float mas = to_b2(mx[u]), mos = to_b2(mo[u]), sh = use_corr ? c1[u] : -c1[u];
            float out = 0.f;
            if (t_main[u]) out += ex2((bs[u] + mas + f0[u]) + c0[u]);
            if (t_prev[u]) out += ex2(bp[u] + mos + mas + (f1[u] + sh));
            if (t_last[u]) out += ex2((bs[u] + mas) + c0[u]);
            if (t_leaf[u]) out += ex2(bs[u] + mas + mos + (f1[u] + sh));
            if (!(out == out)) out = 0.f;
            mg[i] = g * out;
        }
    }
}

// Rule posteriors from the outside weights: lg[a][k][c] = g * sum_{t=1}^{n-1} exp(links[a][k][c] + Wk[a][t] + R[c][t]),
// the one step of the path with operand reuse: per sentence and left option a [Mc,T] x [T,Mc] contraction, which as one
// exponential per term is 9 M exponentials per sentence of 256 main-chain nodes and 140 target tokens.  Here the terms are
// factored, 2^(A) * sum_t 2^(W_t[a] - u_t) * 2^(R_t[c] + corr_t + u_t), and the sum over t runs on the matrix cores in
// fp32 (v_mfma_f32_32x32x2_f32): 0.6 M exponentials per sentence and 36 MFLOP.
//
// One workgroup of four waves per 32x32 tile of (parent, child) pairs with child tile >= parent tile.  The tile's rows
// of the three tables (outside weights of both left options, inside scores) are brought into LDS as base-2 logarithms,
// up to LG_SPAN target positions at a time and all loads of a span in flight together (the tables come from other
// compute units' stores, microseconds away); each wave then takes a quarter of the positions: it exponentiates its
// operands on the way from LDS to the matrix instruction and keeps a partial sum of the whole tile, the four partial
// sums being added through LDS at the end.  Range: the tables vary by hundreds of units along t and along the nodes,
// and only their sums are bounded (a posterior is at most 1).  Per position t the tile's largest outside weight wmax_t
// and largest inside score rmax_t give E_t = wmax_t + rmax_t, and the shift u_t = (wmax_t - rmax_t) / 2 makes both
// factors at most 2^(E_t / 2).  Where every pair of the tile is a rule (child tile behind the parent tile)
// E_t + A <= 0, so nothing overflows and a term that underflows is worth less than 2^(-126 + E_t / 2 - A) of a
// posterior.  In the tiles on the diagonal the two maxima may belong to a pair that is no rule and E_t grows with the
// tile (which is why the tiles are 32 wide); a tile with E_t above range_limit (120 by default: factors below 2^60,
// terms lost only below 2^-40 of a posterior for rules down to 2^-26) is recomputed by its workgroup as one exponential
// per term, which is exact over the whole range (the log-domain form the sweeps use).
// The slab has been zero-filled beforehand.  use_corr: the outside tables are relative to offsets of their own (sweeps
// side by side) and every column takes its correction corr_t.  Dynamic LDS: 3 * 32 * (span + 1) + span floats (and at
// least the 3 * 64 * 17 of the partial sums), span = the number of positions staged at a time (a multiple of 8, at most
// LG_SPAN).
typedef float floatx16 __attribute__((ext_vector_type(16)));
constexpr int LG_TILE = 32, LG_SPAN = 256;
constexpr size_t LG_PART_BYTES = (size_t)3 * 64 * 17 * sizeof(float);  // the partial sums of three waves, one accumulator set
inline size_t links_grad_lds_bytes(int span) {
    const size_t tables = ((size_t)3 * LG_TILE * (span + 1) + span) * sizeof(float);
    return tables > LG_PART_BYTES ? tables : LG_PART_BYTES;
}
// Positions staged at a time, as (span, variant): all of them (up to LG_SPAN, two workgroups to a compute unit: the
// registers that hold a span in flight) while the live tiles fit the device in one round; beyond that equal spans of at
// most LG_SPAN_SMALL with the variant that keeps fewer loads in flight and lets three workgroups share a compute unit.
constexpr int LG_SPAN_SMALL = 96;
inline int links_grad_span(int T, long tiles_live, bool &small) {
    const int all = T - 1 >= LG_SPAN ? LG_SPAN : ((T - 1 + 7) / 8) * 8;
    small = all > LG_SPAN_SMALL && tiles_live > 2L * device_compute_units();
    if (!small) return all;
    const int stages = (T - 1 + LG_SPAN_SMALL - 1) / LG_SPAN_SMALL;
    return (((T - 1 + stages - 1) / stages) + 7) / 8 * 8;
}
template <int QMAX>  // the span is at most 32 * QMAX positions
__global__ __launch_bounds__(256, QMAX < 8 ? 3 : 2) void links_grad_ml1_stream_kernel(const float *__restrict__ grad_out, const float *__restrict__ S,
                                                                   const float *__restrict__ aux_c, const float *__restrict__ links,
                                                                   const int64_t *__restrict__ out_len,
                                                                   const int64_t *__restrict__ tgt_len, float *__restrict__ lgrad,
                                                                   int L, int T, int Mc, Seed seed, int use_corr, float range_limit,
                                                                   int span, MatchGradArgs emis) {
    extern __shared__ float lg_lds[];
    const int ld = span + 1;                 // row pitch: odd, so that a column of 32 rows falls into 32 banks
    float *sw0 = lg_lds, *sw1 = sw0 + LG_TILE * ld, *ss = sw1 + LG_TILE * ld, *s_u = ss + LG_TILE * ld;  // [32][ld] x 3, [span]
    float (*s_part)[64][17] = reinterpret_cast<float (*)[64][17]>(lg_lds);  // partial sums of waves 1..3, one accumulator set
                                                                            // at a time, over the tables once they are used up
    __shared__ int s_bad;
    const int b = blockIdx.z, at = blockIdx.y, ct = blockIdx.x;
    if (ct < at) {  // no tile of rules here: the sentence's emission posteriors, shared among these workgroups
        if (emis.mgrad != nullptr) {
            const int spare = (int)(gridDim.y * (gridDim.y - 1) / 2);
            match_grad_cells<4>(b, (at * (at - 1) / 2 + ct) * 256 + (int)threadIdx.x, spare * 256, grad_out, S, aux_c, emis.match_all,
                                out_len, tgt_len, emis.mgrad, L, T, Mc, seed, use_corr);
        }
        return;
    }
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *Sb = S + (size_t)b * Mc * (T + 2);
    const float ll = Sb[0];
    if (!(lengths_ok(m, n, L, T) && (ll == ll) && (fabsf(ll) != __builtin_huge_valf()))) return;
    const int mc = m / 2;
    if (at * LG_TILE >= mc || ct * LG_TILE >= mc) return;
    AuxViewStream av(const_cast<float *>(aux_c), b, Mc, T);
    const float *corr = ExchangeView(const_cast<float *>(aux_c), b, Mc, T).corr;  // per column, when the sweeps ran side by side
    const float g = seed_weight(grad_out, b, n, seed);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lk = links + (size_t)b * L * 2 * L;
    float *lg = lgrad + (size_t)b * L * 2 * L;
    if (tid == 0) s_bad = 0;

    // positions t1 .. t1 + span - 1 of the tile's rows into LDS (-inf beyond the sentence): thread (tx, ty) takes the positions
    // tx, tx + 32, ... of the rows ty, ty + 8, ty + 16, ty + 24 of the three tables; every load of the span is issued before
    // the first value is stored, so the span costs one trip to memory
    const int tx = tid & 31, ty = tid >> 5;
    auto stage = [&](int t1) {
        float v0[QMAX][4], v1[QMAX][4], vs[QMAX][4];
#pragma unroll
        for (int q = 0; q < QMAX; q++) {
            if (32 * q < span) {  // uniform
                const int tt = t1 + 32 * q + tx;
                const bool tin = tt <= n - 1;
                const float cr = (tin && use_corr) ? corr[tt] : 0.f;
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    const int ra = at * LG_TILE + ty + 8 * p, rc = ct * LG_TILE + ty + 8 * p;
                    v0[q][p] = (tin && ra < mc) ? av.W0[(size_t)ra * (T + 2) + tt] : NEG_INF_F;
                    v1[q][p] = (tin && ra < mc) ? av.W1[(size_t)ra * (T + 2) + tt] : NEG_INF_F;
                    vs[q][p] = (tin && rc < mc) ? av.SR[(size_t)rc * (T + 2) + tt] + cr : NEG_INF_F;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < QMAX; q++) {
            if (32 * q + tx < span) {
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    sw0[(ty + 8 * p) * ld + 32 * q + tx] = v0[q][p];
                    sw1[(ty + 8 * p) * ld + 32 * q + tx] = v1[q][p];
                    ss[(ty + 8 * p) * ld + 32 * q + tx] = vs[q][p];
                }
            }
        }
    };

    // ---- the contraction on the matrix cores
    const int row = lane & 31, kk = lane >> 5;
    floatx16 acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; r++) acc0[r] = acc1[r] = 0.f;
    for (int t1 = 1; t1 <= n - 1; t1 += span) {
        stage(t1);
        __syncthreads();
        // per position: the largest outside weight of the tile's parents, the largest inside score of its children, the shift
        for (int k = tid; k < span; k += 256) {
            float wmax = NEG_INF_F, rmax = NEG_INF_F;
#pragma unroll 8
            for (int r = 0; r < LG_TILE; r++) {
                wmax = fmaxf(wmax, fmaxf(sw0[r * ld + k], sw1[r * ld + k]));
                rmax = fmaxf(rmax, ss[r * ld + k]);
            }
            const bool empty = wmax == NEG_INF_F || rmax == NEG_INF_F;  // no term at this position
            if (!empty && !(wmax + rmax <= range_limit)) s_bad = 1;
            s_u[k] = empty ? __builtin_nanf("") : 0.5f * (wmax - rmax);
        }
        __syncthreads();
        const int live = min(span, n - t1);  // positions of this span inside the sentence (the rest holds -inf)
        for (int k0 = 8 * wave; k0 < live; k0 += 32) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int k = k0 + 2 * j + kk;
                // a position without a finite factor on one side contributes nothing, whatever the other side holds (it is
                // not bounded there: 0 * inf must not reach the accumulators)
                const float u = s_u[k];
                const bool none = !(u == u);
                const float y = none ? 0.f : ex2(ss[row * ld + k] + u);
                const float x0 = none ? 0.f : ex2(sw0[row * ld + k] - u), x1 = none ? 0.f : ex2(sw1[row * ld + k] - u);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x0, y, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(x1, y, acc1, 0, 0, 0);
            }
        }
        __syncthreads();
    }
    if (!s_bad) {  // uniform: last written before the barrier that ends the loop (or never)
        // the four partial sums, one accumulator set at a time: waves 1..3 hand theirs to wave 0
#pragma unroll
        for (int set = 0; set < 2; set++) {
            if (wave > 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) s_part[wave - 1][lane][r] = set == 0 ? acc0[r] : acc1[r];
            }
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float add = (s_part[0][lane][r] + s_part[1][lane][r]) + s_part[2][lane][r];
                    if (set == 0) acc0[r] += add;
                    else acc1[r] += add;
                }
            }
            __syncthreads();
        }
        if (wave != 0) return;
        // accumulator r of lane l: row (r % 4) + 4 * (l / 32) + 8 * (r / 4), column l % 32 of the tile
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int a_id = at * LG_TILE + (r & 3) + 4 * kk + 8 * (r >> 2), c_id = ct * LG_TILE + row;
            if (a_id < mc && c_id < mc && a_id <= c_id) {
                const int a = 2 * a_id + 1, c = 2 * c_id + 1;
                const float A0 = to_b2(lk[((size_t)a * 2 + 0) * L + c]);
                const float A1 = a_id >= 1 ? to_b2(lk[((size_t)a * 2 + 1) * L + c]) : NEG_INF_F;
                const float v0 = ex2(A0) * acc0[r], v1 = ex2(A1) * acc1[r];
                lg[((size_t)a * 2 + 0) * L + c] = (v0 == v0) ? g * v0 : 0.f;
                lg[((size_t)a * 2 + 1) * L + c] = (v1 == v1) ? g * v1 : 0.f;
            }
        }
        return;
    }

    // ---- a factor left the range: the tile again, one exponential per term (four pairs per thread)
    float A0[4], A1[4], e0[4], e1[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int a_id = at * LG_TILE + ty + 8 * q, c_id = ct * LG_TILE + tx;
        const bool ok = a_id < mc && c_id < mc && a_id <= c_id;
        const int a = 2 * a_id + 1, c = 2 * c_id + 1;
        A0[q] = ok ? to_b2(lk[((size_t)a * 2 + 0) * L + c]) : NEG_INF_F;
        A1[q] = (ok && a_id >= 1) ? to_b2(lk[((size_t)a * 2 + 1) * L + c]) : NEG_INF_F;
        e0[q] = e1[q] = 0.f;
    }
    for (int t1 = 1; t1 <= n - 1; t1 += span) {
        if (t1 + span <= n - 1 || t1 > 1) {  // (a single span is still in LDS)
            __syncthreads();
            stage(t1);
            __syncthreads();
        }
        const int live = min(span, n - t1);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int i = ty + 8 * q;
#pragma unroll 4
            for (int u = 0; u < live; u++) {
                const float sc = ss[tx * ld + u];
                e0[q] += ex2((A0[q] + sw0[i * ld + u]) + sc);
                e1[q] += ex2((A1[q] + sw1[i * ld + u]) + sc);
            }
        }
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int a_id = at * LG_TILE + ty + 8 * q, c_id = ct * LG_TILE + tx;
        if (a_id < mc && c_id < mc && a_id <= c_id) {
            const int a = 2 * a_id + 1, c = 2 * c_id + 1;
            lg[((size_t)a * 2 + 0) * L + c] = (e0[q] == e0[q]) ? g * e0[q] : 0.f;
            lg[((size_t)a * 2 + 1) * L + c] = (e1[q] == e1[q]) ? g * e1[q] : 0.f;
        }
    }
}

// The emission posteriors as a launch of their own: one cell per thread.
__global__ __launch_bounds__(256) void match_grad_ml1_stream_kernel(const float *__restrict__ grad_out, const float *__restrict__ S,
                                                                   const float *__restrict__ aux_c, const float *__restrict__ match_all,
                                                                   const int64_t *__restrict__ out_len,
                                                                   const int64_t *__restrict__ tgt_len, float *__restrict__ mgrad, int L,
                                                                   int T, int Mc, Seed seed, int use_corr) {
    match_grad_cells<1>((int)blockIdx.y, (int)(blockIdx.x * blockDim.x + threadIdx.x), (int)(gridDim.x * blockDim.x), grad_out, S, aux_c,
                        match_all, out_len, tgt_len, mgrad, L, T, Mc, seed, use_corr);
}

}  // namespace
}  // namespace pcfgnat
