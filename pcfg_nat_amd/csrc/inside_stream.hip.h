// One-workgroup-per-sentence sweeps of long graphs (more than 130 nodes): link rows streamed from compact copies in L2.
// The only sweeps beyond 1026 nodes, and the second chance of sentences whose pipelined sweeps gave up.
// Part of inside.hip (one translation unit: the kernels share helpers and the anonymous namespace).
#pragma once
#include "inside_common.hip.h"

namespace pcfgnat {
namespace {

// ------------------------------------------------------------------------------------------------------------
// Streaming variants for longer graphs (Mc > 64; the redo path of the pipelined sweeps up to 512 nodes and the only path
// beyond): same sweeps, but the link
// values are fetched from L2 every step (forward: straight from `links`; backward: from a compact transposed copy
// so that lanes read consecutive parents), rows are processed in tiles of 64, and the row reductions are online
// log-sum-exps over chunks of children.  Rule posteriors are produced by a separate, fully parallel kernel from the
// outside weights the sweep leaves behind.
// All tables are relative to the column offsets described in inside_common.hip.h (natural logarithms here).
// Aux layout per sentence (Mc > 64), log-domain values in base 2 like everything inside these kernels: F0h, F1h, Bh,
// W0, W1, R [Mc][T+2] each, D [T+4], padding to a 16-byte boundary, then the compact link matrices (times log2 e) with
// masked entries already -inf and rows padded to MP = 64*ceil(Mc/64) floats:
// Ac [2][Mc][MP] by parent (Ac[k][a][c]) for the forward sweep and At [2][Mc][MP] by child (At[k][c][a]) for the
// outside sweep, so that the sweeps stream them with unconditional 16-byte loads.  Last comes the exchange area of the
// pipelined sweeps (below): the forward columns as doubles [T+2][MP], the outside weights [T+2][2][MP], the shifts every
// block of 16 nodes chose [MP/16][T+4], and four ints (forward gave up, outside sweep gave up, two unused).
// ------------------------------------------------------------------------------------------------------------
__host__ __device__ inline int stream_mp(int Mc) { return ((Mc + 63) / 64) * 64; }
__host__ __device__ inline size_t stream_planes(int Mc, int T) { return (((size_t)6 * Mc * (T + 2) + (size_t)(T + 4)) + 3) & ~(size_t)3; }
__host__ __device__ inline int corr_len(int T) { return (T + 5) & ~1; }
__host__ __device__ inline size_t exchange_floats(int Mc, int T) {
    const size_t MP = stream_mp(Mc);
    // forward columns + outside weights, block shifts, flags; then, for the sweeps that run side by side: the outside
    // weights as absolute doubles, the outside sweep's block shifts, the two correction rows of the posteriors
    return 4 * MP * (T + 2) + (MP / 16) * (T + 4) + 4 + 4 * MP * (T + 2) + (MP / 16) * (T + 4) + 2 * (size_t)corr_len(T);
}
__host__ __device__ inline size_t aux_stride_stream(int Mc, int T) {
    return stream_planes(Mc, T) + (size_t)4 * Mc * stream_mp(Mc) + exchange_floats(Mc, T);
}
struct AuxViewStream {
    float *F0, *F1, *BETA, *W0, *W1, *SR, *D, *Ac, *At;
    __device__ AuxViewStream(float *aux, int b, int Mc, int T) {
        const size_t plane = (size_t)Mc * (T + 2);
        float *base = aux + (size_t)b * aux_stride_stream(Mc, T);
        F0 = base;
        F1 = base + plane;
        BETA = base + 2 * plane;
        W0 = base + 3 * plane;
        W1 = base + 4 * plane;
        SR = base + 5 * plane;
        D = base + 6 * plane;
        Ac = base + stream_planes(Mc, T);
        At = Ac + (size_t)2 * Mc * stream_mp(Mc);
    }
};
struct ExchangeView {
    unsigned long long *fcol;  // [T+2][MP]
    unsigned *bw;              // [T+2][2][MP]
    float *shifts;             // [MP/16][T+4]
    int *flags;
    unsigned long long *obw;   // [T+2][2][MP]: outside weights as absolute doubles (sweeps side by side)
    float *shiftsE;            // [MP/16][T+4]: shifts of the outside sweep's blocks (sweeps side by side)
    float *corr;               // [2][corr_len(T)]: corrections of the posteriors, corr_t and corr1_t
    __device__ ExchangeView(float *aux, int b, int Mc, int T) {
        const int MP = stream_mp(Mc);
        float *base = aux + (size_t)b * aux_stride_stream(Mc, T) + stream_planes(Mc, T) + (size_t)4 * Mc * MP;
        fcol = reinterpret_cast<unsigned long long *>(base);
        bw = reinterpret_cast<unsigned *>(base + (size_t)2 * MP * (T + 2));
        shifts = base + (size_t)4 * MP * (T + 2);
        flags = reinterpret_cast<int *>(shifts + (size_t)(MP / 16) * (T + 4));
        float *more = shifts + (size_t)(MP / 16) * (T + 4) + 4;
        obw = reinterpret_cast<unsigned long long *>(more);
        shiftsE = more + (size_t)4 * MP * (T + 2);
        corr = shiftsE + (size_t)(MP / 16) * (T + 4);
    }
};
constexpr int FLAG_FWD = 0, FLAG_BWD = 1;

// The streaming sweeps give a node SL lanes (4, 8 or 16), each of which takes four consecutive entries of every chunk of
// 4*SL, and handle NT/SL nodes per pass.  Fewer lanes per node mean fewer passes and reductions per column, more lanes
// mean longer contiguous reads per node.
template <int SL>
__device__ __forceinline__ float node_max(float v) {
    if (SL == 4) return dpp_max_xor2(dpp_max_xor1(v));
    return SL == 8 ? row8_max(v) : row16_max(v);
}
template <int SL>
__device__ __forceinline__ float node_sum(float v) {
    if (SL == 4) {
        v += dpp_f<DPP_QUAD_XOR1>(v);
        v += dpp_f<DPP_QUAD_XOR2>(v);
        return v;
    }
    return SL == 8 ? row8_sum(v) : row16_sum(v);
}

// log2-sum-exp2 with a running maximum, four terms at a time; SL lanes share a row
template <int SL>
struct RunningLse {
    float m, s;
    __device__ RunningLse() : m(NEG_INF_F), s(0.f) {}
    __device__ __forceinline__ void add4(const float4 &a, const float4 &b) {  // folds a + b
        const float v0 = a.x + b.x, v1 = a.y + b.y, v2 = a.z + b.z, v3 = a.w + b.w;
        const float cm = fmaxf(fmaxf(v0, v1), fmaxf(v2, v3));
        if (cm > m) {
            s *= ex2(m - cm);  // m = -inf gives 0 * 0
            m = cm;
        }
        if (m != NEG_INF_F) s += (ex2(v0 - m) + ex2(v1 - m)) + (ex2(v2 - m) + ex2(v3 - m));
    }
    __device__ __forceinline__ void merge(const RunningLse<SL> &o) {
        const float M = fmaxf(m, o.m);
        if (M == NEG_INF_F) return;
        s = s * ex2(m - M) + o.s * ex2(o.m - M);
        m = M;
    }
    // combine the lanes of a node; every lane gets the log2-sum-exp2 of all folded terms
    __device__ __forceinline__ float finish() const {
        const float M = node_max<SL>(m + 0.f);  // the add keeps the reduction's input from being a raw exp/log result
        const float part = (m == NEG_INF_F) ? 0.f : s * ex2(m - M);
        const float tot = node_sum<SL>(part);
        return (M == NEG_INF_F) ? NEG_INF_F : M + lg2(tot);
    }
};

__device__ __forceinline__ float sum4_ex2(const float4 &a, const float4 &b) {
    return (ex2(a.x + b.x) + ex2(a.y + b.y)) + (ex2(a.z + b.z) + ex2(a.w + b.w));
}
__device__ __forceinline__ float4 minus(const float4 &a, float g) { return make_float4(a.x - g, a.y - g, a.z - g, a.w - g); }
__device__ __forceinline__ bool is_finite(float v) { return fabsf(v) < __builtin_huge_valf(); }  // false for NaN too

// Base-2 log-sum-exp of one node's two link rows r0, r1 (SL lanes per node, each lane four consecutive entries of every
// chunk q in [q0, q1)) against LDS columns: out0 = LSE_i(r0[i] + u0[i]), out1 = LSE_i(r1[i] + u1[i]), or with
// JOINT the one value LSE over both in out0; has1 = false says that r1 is known to be all -inf.  The terms are first
// summed relative to a guess g of the results (the node's out0 one column earlier, which differs from the new one by about
// one token's log-probability and from out1 by about one link's).  A sum is accepted when it
// lies in [2^-90, 2^100]: then no term overflowed and the terms flushed to zero are below 2^-126 each, i.e. far below
// rounding.  Otherwise (no derivation at all, first columns, a guess that is far off) the rows are read again and
// folded with a running maximum, which is exact for any input.  Link values are requested one chunk ahead: x0, x1 hold
// the row's first chunk on entry and, on exit, the chunk at n0, n1 (the first chunk of the row this lane handles next).
template <bool JOINT, int SL>
__device__ __forceinline__ void stream_row_lse(const float4 *__restrict__ r0, const float4 *__restrict__ r1, const float4 *u0,
                                               const float4 *u1, int q0, int q1, bool live, bool has1, float g, float4 &x0, float4 &x1, const float4 *__restrict__ n0,
                                               const float4 *__restrict__ n1, float &out0, float &out1) {
    g = is_finite(g) ? g : 0.f;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll 2
    for (int q = q0; q + 1 < q1; q++) {
        const float4 y0 = x0, y1 = x1;
        x0 = r0[SL * (q + 1)];
        x1 = r1[SL * (q + 1)];
        const float4 c0 = minus(u0[SL * q], g);
        const float4 c1 = JOINT ? minus(u1[SL * q], g) : c0;
        s0 += sum4_ex2(y0, c0);
        s1 += sum4_ex2(y1, c1);
    }
    {   // last chunk of this node, first chunk of the next one requested
        const float4 y0 = x0, y1 = x1;
        x0 = *n0;
        x1 = *n1;
        const float4 c0 = minus(u0[SL * (q1 - 1)], g);
        const float4 c1 = JOINT ? minus(u1[SL * (q1 - 1)], g) : c0;
        s0 += sum4_ex2(y0, c0);
        s1 += sum4_ex2(y1, c1);
    }
    bool ok;
    if (JOINT) {
        const float tot = node_sum<SL>(s0 + s1);
        ok = tot >= 0x1p-90f && tot <= 0x1p100f;
        out0 = g + lg2(tot);
        out1 = out0;
    } else {
        const float t0 = node_sum<SL>(s0), t1 = node_sum<SL>(s1);
        ok = t0 >= 0x1p-90f && t0 <= 0x1p100f && ((t1 >= 0x1p-90f && t1 <= 0x1p100f) || !has1);
        out0 = g + lg2(t0);
        out1 = has1 ? g + lg2(t1) : NEG_INF_F;
    }
    if (live && !ok) {  // uniform over the lanes of the node
        RunningLse<SL> a0, a1;
        for (int q = q0; q < q1; q++) {
            const float4 c0 = u0[SL * q];
            const float4 c1 = JOINT ? u1[SL * q] : c0;
            a0.add4(r0[SL * q], c0);
            a1.add4(r1[SL * q], c1);
        }
        if (JOINT) {
            a0.merge(a1);
            out0 = out1 = a0.finish();
        } else {
            out0 = a0.finish();
            out1 = a1.finish();
        }
    }
}

// Dynamic LDS: col[2][MP], f1prev[MP], f0prev[MP], per-wave column maxima slots[2][16], then (if MATCH_LDS) match main
// [Mc][T], match leaf [Mc][T].
// (sentence b by one workgroup of NT threads; the kernels below run it)
template <bool MATCH_LDS, int SL>
__device__ __forceinline__ void inside_fwd_ml1_stream_block(const int b, const float *__restrict__ match_all,
                                                            const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                            const int64_t *__restrict__ tgt_len, float *__restrict__ S,
                                                            float *__restrict__ aux, int L, int T, int Mc, int MP, float *smem) {
    float *col = smem;               // [2][MP]
    float *f1prev = smem + 2 * MP;    // [MP]
    float *f0prev = smem + 3 * MP;    // [MP]  (only a guess for the next column)
    float *slots = smem + 4 * MP;     // [2][16]
    float *sm_main = slots + 32;      // [Mc][T]
    float *sm_leaf = sm_main + (MATCH_LDS ? Mc * T : 0);

    constexpr int SCH = 4 * SL, SROWS = NT / SL;
    const int tid = threadIdx.x, gidx = tid / SL, j = tid % SL;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    float *Sb = S + (size_t)b * Mc * (T + 2);
    AuxViewStream av(aux, b, Mc, T);

    if (!lengths_ok(m, n, L, T)) {
        for (int i = tid; i < Mc * (T + 2); i += NT) Sb[i] = (i == 0) ? __builtin_nanf("") : NEG_INF_F;
        return;
    }
    const int mc = m / 2;
    if (MATCH_LDS) {
        for (int i = tid; i < Mc * T; i += NT) {
            const int a_id = i / T, s = i - a_id * T;
            const bool ok = a_id < mc && s < n;
            sm_main[i] = ok ? to_b2(mt[(size_t)(2 * a_id + 1) * T + s]) : NEG_INF_F;
            sm_leaf[i] = (ok && a_id >= 1) ? to_b2(mt[(size_t)(2 * a_id) * T + s]) : NEG_INF_F;
        }
    }
    for (int i = tid; i < Mc * (T + 2); i += NT) {
        const int a_id = i / (T + 2), s = i - a_id * (T + 2);
        if (a_id >= mc || s >= n - 1) {
            float v = NEG_INF_F;
            if (a_id == mc - 1 && s == n - 1) v = sanitize(mt[(size_t)(m - 1) * T + (n - 1)]);
            Sb[i] = v;
            av.SR[i] = v * LOG2E_F;
        }
    }
    const float base_cell = to_b2(mt[(size_t)(m - 1) * T + (n - 1)]);
    for (int i = tid; i < MP; i += NT) {
        col[((n - 1) & 1) * MP + i] = (i == mc - 1) ? base_cell : NEG_INF_F;
        col[((n - 2) & 1) * MP + i] = NEG_INF_F;
        f1prev[i] = NEG_INF_F;
        f0prev[i] = NEG_INF_F;
    }
    if (tid < 32) slots[tid] = base_cell;  // maximum of column n-1
    for (int i = tid; i < T + 4; i += NT) av.D[i] = 0.f;
    __syncthreads();

    const int ntiles = (mc + SROWS - 1) / SROWS, nq = (mc + SCH - 1) / SCH;
    // What a lane needs from memory for node tile*SROWS+gidx at step t, requested one node ahead (across the step's
    // barrier too: none of it depends on the column being computed).  q0 = the chunk that holds the node's diagonal, the
    // same for all nodes of a wave.
    struct Ahead {
        const float4 *r0, *r1;
        float ma_p, ml_p, ma_t;
        int q0;
    };
    auto look_ahead = [&](int tile, int t) -> Ahead {
        const int a_id = tile * SROWS + gidx;
        const int ar = a_id < mc ? a_id : Mc - 1;  // rows beyond the sentence: any valid address, the result is discarded
        Ahead h;
        h.q0 = min(__builtin_amdgcn_readfirstlane(a_id / SCH), nq - 1);
        h.r0 = reinterpret_cast<const float4 *>(av.Ac + ((size_t)0 * Mc + ar) * MP) + j;
        h.r1 = reinterpret_cast<const float4 *>(av.Ac + ((size_t)1 * Mc + ar) * MP) + j;
        if (MATCH_LDS) {
            h.ma_p = sm_main[ar * T + t - 1];
            h.ml_p = sm_leaf[ar * T + t - 1];
            h.ma_t = sm_main[ar * T + t];
        } else {
            const float *ra = mt + (size_t)(2 * ar + 1) * T, *rl = mt + (size_t)(2 * ar) * T;
            h.ma_p = to_b2(ra[t - 1]);
            h.ml_p = ar >= 1 ? to_b2(rl[t - 1]) : NEG_INF_F;
            h.ma_t = to_b2(ra[t]);
        }
        return h;
    };
    Ahead nx = look_ahead(0, n - 1);
    float4 x0 = nx.r0[SL * nx.q0], x1 = nx.r1[SL * nx.q0];
    double O = 0.0;  // offset of the column being read
    for (int t = n - 1; t >= 1; t--) {
        const float *cur = col + (t & 1) * MP;
        float *nxt = col + ((t - 1) & 1) * MP;
        const float D = fmaxf(max8(slots + (t & 1) * 16), max8(slots + (t & 1) * 16 + 8));
        const float Ds = (D == NEG_INF_F) ? 0.f : D;
        const double O_new = O + (double)Ds;
        float wmax = NEG_INF_F;
        for (int tile = 0; tile < ntiles; tile++) {
            const int a_id = tile * SROWS + gidx;
            const bool row_ok = a_id < mc;
            const Ahead me = nx;
            const bool last_tile = tile + 1 == ntiles;
            nx = look_ahead(last_tile ? 0 : tile + 1, (last_tile && t > 1) ? t - 1 : t);
            // children c >= a, from the chunk that holds the diagonal
            const float4 *cv = reinterpret_cast<const float4 *>(cur) + j;
            const int ai = min(a_id, MP - 1);  // the last tile may reach beyond the padded node count
            const float f1p = f1prev[ai];
            float F0, F1;
            stream_row_lse<false, SL>(me.r0, me.r1, cv, cv, me.q0, nq, row_ok, a_id >= 1, f0prev[ai], x0, x1, nx.r0 + SL * nx.q0,
                                  nx.r1 + SL * nx.q0, F0, F1);
            F0 -= Ds;
            F1 -= Ds;
            float s_new = lse2_b2(me.ma_p + F0, (me.ml_p + me.ma_t) + (f1p - Ds));
            if (!row_ok) s_new = NEG_INF_F;
            wmax = fmaxf(wmax, s_new);
            if (j == 0 && a_id < MP) {
                nxt[a_id] = s_new;
                f1prev[a_id] = F1;
                f0prev[a_id] = F0;
                if (row_ok) {
                    Sb[(size_t)a_id * (T + 2) + (t - 1)] = (float)(((double)s_new + O_new) * LN2_D);
                    av.SR[(size_t)a_id * (T + 2) + (t - 1)] = s_new;
                    av.F0[(size_t)a_id * (T + 2) + t] = F0;
                    av.F1[(size_t)a_id * (T + 2) + t] = F1;
                }
            }
        }
        {
            const float wm = wave_max(wmax);
            if ((tid & 63) == 0) slots[((t - 1) & 1) * 16 + (tid >> 6)] = wm;
        }
        if (tid == 0) av.D[t] = Ds;
        O = O_new;
        lds_barrier();
    }
}

template <bool MATCH_LDS, int SL>
__global__ __launch_bounds__(NT) void inside_fwd_ml1_stream_kernel(const float *__restrict__ match_all, const float *__restrict__ links,
                                                                  const int64_t *__restrict__ out_len,
                                                                  const int64_t *__restrict__ tgt_len, float *__restrict__ S,
                                                                  float *__restrict__ aux, int L, int T, int Mc, int MP,
                                                                  int only_flagged) {
    // only_flagged: run only for sentences whose pipelined sweep gave up (the flag was written by an earlier launch)
    if (only_flagged) {
        if (ExchangeView(aux, blockIdx.x, Mc, T).flags[FLAG_FWD] == 0) return;
        if (threadIdx.x == 0) atomicAdd(&g_inside_redone, 1ull);
    }
    extern __shared__ float smem[];
    inside_fwd_ml1_stream_block<MATCH_LDS, SL>((int)blockIdx.x, match_all, links, out_len, tgt_len, S, aux, L, T, Mc, MP, smem);
}

// Compact copies of the main-chain links for the streaming sweeps: Ac[k][a_id][c_id] = At[k][c_id][a_id] =
// log2(e) * links[2*a_id+1][k][2*c_id+1] where a_id <= c_id < mc (k = 1 needs a_id >= 1), -inf everywhere else including the
// padding columns up to MP.  One block per 32 x 32 tile of (parent, child) pairs, grid (MP/32, MP/32, B).  The blocks of a
// sentence also share the filling of its exchange tables and, when the caller hands one over (single call), the zero fill of
// the sentence's slab of links_grad (2 L^2 floats), which the posterior kernel only writes at its posterior cells.
__global__ __launch_bounds__(256) void compact_links_ml1_kernel(const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                               float *__restrict__ aux, int L, int T, int Mc, int MP,
                                                               float *__restrict__ zero_slabs) {
    __shared__ float tile[2][32][33];
    const int b = blockIdx.z;
    if (zero_slabs != nullptr) {
        float *z = zero_slabs + (size_t)b * L * 2 * L;
        const size_t nthreads = (size_t)gridDim.x * gridDim.y * 256, me = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        const size_t nz = (size_t)L * 2 * L;
        if ((reinterpret_cast<uintptr_t>(z) & 15) == 0) {  // 16 bytes per store where the slab allows it
            float4 *z4 = reinterpret_cast<float4 *>(z);
            for (size_t i = me; i < nz / 4; i += nthreads) z4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (me < (nz & 3)) z[(nz & ~(size_t)3) + me] = 0.f;
        } else {
            for (size_t i = me; i < nz; i += nthreads) z[i] = 0.f;
        }
    }
    const int m = (int)out_len[b];
    const int mc = (m >= 2 && m <= L) ? m / 2 : 0;
    AuxViewStream av(aux, b, Mc, T);
    const float *lk = links + (size_t)b * L * 2 * L;
    const int a0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    {   // the exchange tables of the pipelined sweeps start out empty (all ones), their flags lowered
        ExchangeView xv(aux, b, Mc, T);
        // both tables start 16-byte aligned and hold a multiple of four words (MP is a multiple of 64)
        uint4 *x = reinterpret_cast<uint4 *>(xv.fcol), *y = reinterpret_cast<uint4 *>(xv.obw);
        const size_t quads = (size_t)MP * (T + 2);
        const size_t nthreads = (size_t)gridDim.x * gridDim.y * 256, me = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        const uint4 ones = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
        for (size_t i = me; i < quads; i += nthreads) {
            x[i] = ones;
            y[i] = ones;
        }
        if (me < 4) xv.flags[me] = 0;
    }
    for (int r = ty; r < 32; r += 8) {
        const int a_id = a0 + r, c_id = c0 + tx;
        const bool ok = a_id < mc && c_id < mc && a_id <= c_id;
        const size_t row = (size_t)(2 * a_id + 1) * 2;
        const float x0 = ok ? to_b2(lk[(row + 0) * L + 2 * c_id + 1]) : NEG_INF_F;
        const float x1 = (ok && a_id >= 1) ? to_b2(lk[(row + 1) * L + 2 * c_id + 1]) : NEG_INF_F;
        tile[0][r][tx] = x0;
        tile[1][r][tx] = x1;
        if (a_id < Mc) {
            av.Ac[((size_t)0 * Mc + a_id) * MP + c_id] = x0;
            av.Ac[((size_t)1 * Mc + a_id) * MP + c_id] = x1;
        }
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        const int c_id = c0 + r, a_id = a0 + tx;
        if (c_id < Mc) {
            av.At[((size_t)0 * Mc + c_id) * MP + a_id] = tile[0][tx][r];
            av.At[((size_t)1 * Mc + c_id) * MP + a_id] = tile[1][tx][r];
        }
    }
}

// Outside sweep.  Dynamic LDS: w0[2][MP], w1[2][MP], bprev[MP], D[T+4], then (if MATCH_LDS) match main/leaf [Mc][T] each.
// (sentence b by one workgroup of NT threads; the kernels below run it)
template <bool MATCH_LDS, int SL>
__device__ __forceinline__ void inside_bwd_ml1_stream_block(const int b, const float *__restrict__ S, float *__restrict__ aux,
                                                            const float *__restrict__ match_all, const int64_t *__restrict__ out_len,
                                                            const int64_t *__restrict__ tgt_len, int L, int T, int Mc, int MP,
                                                            float *smem) {
    float *w0 = smem;             // [2][MP]
    float *w1 = smem + 2 * MP;     // [2][MP]
    float *bprev = smem + 4 * MP;  // [MP]
    float *sm_D = smem + 5 * MP;   // [T+4]
    float *sm_main = sm_D + (T + 4);
    float *sm_leaf = sm_main + (MATCH_LDS ? Mc * T : 0);

    constexpr int SCH = 4 * SL, SROWS = NT / SL;
    const int tid = threadIdx.x, gidx = tid / SL, j = tid % SL;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *Sb = S + (size_t)b * Mc * (T + 2);
    AuxViewStream av(aux, b, Mc, T);
    const float ll = Sb[0];
    const bool valid = lengths_ok(m, n, L, T) && (ll == ll) && (fabsf(ll) != __builtin_huge_valf());
    if (!valid) return;  // the posterior kernels write zeros for such sentences
    const int mc = m / 2;
    if (MATCH_LDS) {
        for (int i = tid; i < Mc * T; i += NT) {
            const int a_id = i / T, s = i - a_id * T;
            const bool ok = a_id < mc && s < n;
            sm_main[i] = ok ? to_b2(mt[(size_t)(2 * a_id + 1) * T + s]) : NEG_INF_F;
            sm_leaf[i] = (ok && a_id >= 1) ? to_b2(mt[(size_t)(2 * a_id) * T + s]) : NEG_INF_F;
        }
    }
    for (int i = tid; i < T + 4; i += NT) sm_D[i] = av.D[i];
    __syncthreads();
    auto match_main = [&](int a_id, int s) -> float {
        if (MATCH_LDS) return sm_main[a_id * T + s];
        return to_b2(mt[(size_t)(2 * a_id + 1) * T + s]);
    };
    auto match_leaf = [&](int a_id, int s) -> float {
        if (MATCH_LDS) return sm_leaf[a_id * T + s];
        return a_id >= 1 ? to_b2(mt[(size_t)(2 * a_id) * T + s]) : NEG_INF_F;
    };
    const float beta00 = -av.SR[0];  // relative to the offset of column 0
    const float w00 = (match_main(0, 0) + beta00) - sm_D[1];
    for (int i = tid; i < MP; i += NT) {
        w0[1 * MP + i] = (i == 0) ? w00 : NEG_INF_F;
        w1[1 * MP + i] = NEG_INF_F;
        w0[0 * MP + i] = NEG_INF_F;
        w1[0 * MP + i] = NEG_INF_F;
        bprev[i] = (i == 0) ? beta00 : NEG_INF_F;
    }
    for (int i = tid; i < mc; i += NT) {
        av.BETA[(size_t)i * (T + 2)] = (i == 0) ? beta00 : NEG_INF_F;
        av.W0[(size_t)i * (T + 2) + 1] = (i == 0) ? w00 : NEG_INF_F;
        av.W1[(size_t)i * (T + 2) + 1] = NEG_INF_F;
    }
    __syncthreads();

    const int ntiles = (mc + SROWS - 1) / SROWS, nq = (mc + SCH - 1) / SCH;
    // what a lane needs from memory for node tile*SROWS+gidx at step t, requested one node ahead; q1 = one past the chunk
    // that holds the node's diagonal, the same for all nodes of a wave
    struct Ahead {
        const float4 *r0, *r1;
        float mc_t, ml_p;
        int q1;
    };
    auto look_ahead = [&](int tile, int t) -> Ahead {
        const int c_id = tile * SROWS + gidx;
        const bool live = c_id < mc;
        const int ci = live ? c_id : 0;
        Ahead h;
        h.q1 = min(__builtin_amdgcn_readfirstlane(c_id / SCH), nq - 1) + 1;
        h.r0 = reinterpret_cast<const float4 *>(av.At + ((size_t)0 * Mc + ci) * MP) + j;
        h.r1 = reinterpret_cast<const float4 *>(av.At + ((size_t)1 * Mc + ci) * MP) + j;
        h.mc_t = live ? match_main(ci, t) : NEG_INF_F;
        h.ml_p = live ? match_leaf(ci, t - 1) : NEG_INF_F;
        return h;
    };
    Ahead nx = look_ahead(0, 1);
    float4 x0 = nx.r0[0], x1 = nx.r1[0];
    for (int t = 1; t <= n - 1; t++) {
        const float *c0 = w0 + (t & 1) * MP, *c1 = w1 + (t & 1) * MP;
        float *n0 = w0 + ((t + 1) & 1) * MP, *n1 = w1 + ((t + 1) & 1) * MP;
        const float d_next = sm_D[t + 1], d_both = d_next + sm_D[t];
        for (int tile = 0; tile < ntiles; tile++) {
            const int c_id = tile * SROWS + gidx;
            const bool live = c_id < mc;
            const Ahead me = nx;
            const bool last_tile = tile + 1 == ntiles;
            nx = look_ahead(last_tile ? 0 : tile + 1, (last_tile && t < n - 1) ? t + 1 : t);
            const float mc_t = me.mc_t, ml_p = me.ml_p;
            // parents a <= c, up to the chunk that holds the diagonal
            const float4 *u0 = reinterpret_cast<const float4 *>(c0) + j, *u1 = reinterpret_cast<const float4 *>(c1) + j;
            const float bp = bprev[min(c_id, MP - 1)];  // the last tile may reach beyond the padded node count
            float beta, unused;
            stream_row_lse<true, SL>(me.r0, me.r1, u0, u1, 0, me.q1, live, true, bp, x0, x1, nx.r0, nx.r1, beta, unused);
            if (!live) beta = NEG_INF_F;
            const float nw0 = (mc_t + beta) - d_next;
            const float nw1 = ((ml_p + mc_t) + bp) - d_both;
            if (j == 0 && c_id < MP) {
                n0[c_id] = nw0;
                n1[c_id] = nw1;
                bprev[c_id] = beta;
                if (live) {
                    av.BETA[(size_t)c_id * (T + 2) + t] = beta;
                    av.W0[(size_t)c_id * (T + 2) + t + 1] = nw0;
                    av.W1[(size_t)c_id * (T + 2) + t + 1] = nw1;
                }
            }
        }
        lds_barrier();
    }
}

}  // namespace
}  // namespace pcfgnat
