// Inside and outside sweeps of graphs of up to 130 nodes (one workgroup of 512 threads per sentence and sweep, link slabs in
// registers): the kernels of the two-call API, the fused single launch, the paired sweeps of the single call with the
// pad-row fill beside them, and the kernel that multiplies their tables into the posteriors.
// Part of inside.hip (one translation unit: the kernels share helpers and the anonymous namespace).
#pragma once
#include "inside_common.hip.h"

namespace pcfgnat {
namespace {

// ------------------------------------------------------------------------------------------------------------
// Register-resident sweeps (Mc <= 64 in use; the kernels take up to 128 nodes with R = 2).  512 threads = 8 waves; a node is owned by an 8-lane group (two groups per DPP
// row), the 8 lanes stride over the other index in chunks of 8.  Link slabs are triangular (children c >= a), so wave w
// takes node block perm(w) = {0,1,2,3,7,6,5,4}[w] of every 64-node tile: the two waves that share a SIMD (w, w+4) then
// own blocks p and 7-p and together always process 9 of the 16 chunks, whole chunks below the diagonal being skipped
// with wave-uniform branches.  All log-domain quantities are held in base 2 (pre-multiplied by log2 e) so that the
// hardware exp2/log2 are used without extra multiplies; tables that leave the kernel in the reference's layout (S) are
// converted back on store, the private auxiliary tables (F0, F1, BETA) stay in base 2.
// ------------------------------------------------------------------------------------------------------------
constexpr int NTR = 512;
constexpr size_t LDS_BUDGET = 128 * 1024;  // of the 160 KB a gfx950 workgroup may use
constexpr float LOG2E_F = 1.4426950408889634f;
constexpr double LN2_D = 0.6931471805599453094;

// Diagnostic: sweeps (forward or outside, counted apart) that the one-workgroup kernels redid because the pipelined
// sweep of the sentence gave up, since the library was loaded (pcfgnat_pipeline_redo_counts).
__device__ unsigned long long g_inside_redone;
// Diagnostic: sentences given up for good - both pipelined sweeps gave up AND the outside sweep's second chance outwaited
// its bound for the forward's (seconds; pcfgnat_pipeline_redo_wait_limit).  Their log-likelihood is NaN, which the
// criterion counts as an invalid sentence: never a wrong gradient, and never unnoticed, thanks to this counter.
__device__ unsigned long long g_inside_given_up;

__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float lg2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float to_b2(float natural) { return sanitize(natural) * LOG2E_F; }


__device__ __forceinline__ float row8_max(float v) {
    v = dpp_max_xor1(v);
    v = dpp_max_xor2(v);
    v = dpp_max_half_mirror(v);
    return v;
}
__device__ __forceinline__ float row8_sum(float v) {
    v += dpp_f<DPP_QUAD_XOR1>(v);
    v += dpp_f<DPP_QUAD_XOR2>(v);
    v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
    return v;
}
__device__ __forceinline__ float lse2_b2(float a, float b) {
    const float m = fmaxf(a, b);
    if (m == NEG_INF_F) return NEG_INF_F;
    return m + lg2(ex2(a - m) + ex2(b - m));
}
// node block of wave w inside a 64-node tile (wave-uniform scalar)
__device__ __forceinline__ int wave_block(int wave) { return __builtin_amdgcn_readfirstlane(wave < 4 ? wave : 11 - wave); }

struct FwdSweepArgs {
    float *col, *sm_main, *sm_leaf, *sm_S, *sm_F0, *sm_F1;
    const float *mt;
    float *Sb, *gF0, *gF1, *gSR;
    float *slots, *sm_D;
    double *sm_O;
    float base_b2;  // the base cell S[last][n-1], base 2
    int n, mc, Mc, T, j, g8;
};

// max of three values that need no canonicalisation (loaded from tables this kernel wrote)
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// maximum of eight floats stored at a 16-byte aligned LDS address (two broadcast reads)
__device__ __forceinline__ float max8(const float *p) {
    const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
    return max3_raw(max3_raw(a.x, a.y, a.z), max3_raw(a.w, b.x, b.y), max3_raw(b.z, b.w, b.w));
}
// maximum over the wave of a value that is uniform inside each 8-lane group
__device__ __forceinline__ float wave_max_of_groups(float v) {
    v = dpp_max_mirror(v);
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// The forward sweep of one wave, specialised on its node block P so that the chunks below the diagonal (q < 8r + P)
// vanish at compile time.  Executes n-1 workgroup barriers regardless of P.
template <int R, bool TAB_LDS, int P>
__device__ __forceinline__ void fwd_sweep(const float (&A0)[R][8 * R], const float (&A1)[R][8 * R], const FwdSweepArgs &x) {
    constexpr int NQ = 8 * R;
    constexpr int MP = 64 * R;
    const int T = x.T, TS = x.T + 2, j = x.j;
    float F1prev[R];
    float wprev = x.base_b2;  // this wave's maximum of the column written by the previous step
#pragma unroll
    for (int r = 0; r < R; r++) F1prev[r] = NEG_INF_F;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    double O = 0.0;  // offset of the column being read
    for (int t = x.n - 1; t >= 1; t--) {
        const float *cur = x.col + (t & 1) * MP;
        float *nxt = x.col + ((t - 1) & 1) * MP;
        float wmax = NEG_INF_F;
        float Ds = 0.f;
        double O_new = 0.0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int a_id = 64 * r + 8 * P + x.g8;
            const int q0 = 8 * r + P;  // chunks below hold only children c < a
            const int ai = (a_id < x.Mc) ? a_id : 0;
            float sc[NQ];
#pragma unroll
            for (int q = 0; q < NQ; q++)
                if (q >= q0) sc[q] = cur[j + 8 * q];
            if (r == 0) {
                // Bookkeeping in the shadow of the column loads (issued after them on purpose).  Shift of this step: the
                // maximum of column t+1, whose per-wave parts were published one step ago.  (LDS float-max atomics on
                // one cell would give the maximum of column t itself without the reduction below, but 64 of them per
                // step on one address cost ten times more than this.)
                const float D = max8(x.slots + ((t + 1) & 1) * 8);
                x.slots[(t & 1) * 8 + wave] = wave_max_of_groups(wprev);  // maximum of column t, read by step t-1
                Ds = (D == NEG_INF_F) ? 0.f : D;
                if (!TAB_LDS || wave == 0) O_new = O + (double)Ds;  // offset of column t-1
                if (wave == 0) {
                    x.sm_D[t] = Ds;
                    x.sm_O[t - 1] = O_new;
                }
            }
            float ma_p, ml_p, ma_t;  // match[a][t-1], match[a-1][t-1], match[a][t]
            if (TAB_LDS) {
                ma_p = x.sm_main[ai * T + t - 1];
                ml_p = x.sm_leaf[ai * T + t - 1];
                ma_t = x.sm_main[ai * T + t];
            } else {
                const size_t ra = (size_t)(2 * ai + 1) * T, rl = (size_t)(2 * ai) * T;
                const float x0 = x.mt[ra + t - 1], x1 = x.mt[rl + t - 1], x2 = x.mt[ra + t];
                const bool ok = a_id < x.mc;
                ma_p = ok ? to_b2(x0) : NEG_INF_F;
                ml_p = (ok && a_id >= 1) ? to_b2(x1) : NEG_INF_F;
                ma_t = ok ? to_b2(x2) : NEG_INF_F;
            }
            float v0[NQ], v1[NQ];
            float m0 = NEG_INF_F, m1 = NEG_INF_F;
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q >= q0) {
                    v0[q] = A0[r][q] + sc[q];
                    v1[q] = A1[r][q] + sc[q];
                    m0 = fmaxf(m0, v0[q]);
                    m1 = fmaxf(m1, v1[q]);
                }
            }
            m0 = row8_max(m0);
            m1 = row8_max(m1);
            const float m0s = (m0 == NEG_INF_F) ? 0.f : m0, m1s = (m1 == NEG_INF_F) ? 0.f : m1;
            float e0 = 0.f, e1 = 0.f;
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q >= q0) {
                    e0 += ex2(v0[q] - m0s);
                    e1 += ex2(v1[q] - m1s);
                }
            }
            e0 = row8_sum(e0);
            e1 = row8_sum(e1);
            const float F0 = (m0 == NEG_INF_F) ? NEG_INF_F : (m0 - Ds) + lg2(e0);
            const float F1 = (m1 == NEG_INF_F) ? NEG_INF_F : (m1 - Ds) + lg2(e1);
            float s_new = lse2_b2(ma_p + F0, (ml_p + ma_t) + (F1prev[r] - Ds));
            if (a_id >= x.mc) s_new = NEG_INF_F;
            F1prev[r] = F1;
            wmax = fmaxf(wmax, s_new);
            if (j == 0) {
                nxt[a_id] = s_new;
                if (a_id < x.mc) {
                    if (TAB_LDS) {
                        x.sm_S[a_id * TS + (t - 1)] = s_new;
                        x.sm_F0[a_id * TS + t] = F0;
                        x.sm_F1[a_id * TS + t] = F1;
                    } else {
                        x.Sb[(size_t)a_id * TS + (t - 1)] = (float)(((double)s_new + O_new) * LN2_D);
                        x.gSR[(size_t)a_id * TS + (t - 1)] = s_new;
                        x.gF0[(size_t)a_id * TS + t] = F0;
                        x.gF1[(size_t)a_id * TS + t] = F1;
                    }
                }
            }
        }
        wprev = wmax;
        O = O_new;
        lds_barrier();
    }
}

// Forward.  Dynamic LDS: head (see LdsHead), col[2][64R]; with TAB_LDS also the emissions of main nodes and of their
// leaves [Mc][T] and the R, F0h, F1h tables [Mc][T+2] (all base 2), which are copied out in bulk when the sweep is over -
// the sweep itself then touches no global memory.
template <int R, bool TAB_LDS>
__device__ __forceinline__ void inside_fwd_ml1_body(const int b, const float *__restrict__ match_all, const float *__restrict__ links,
                                                   const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                   float *__restrict__ S, float *__restrict__ aux, int L, int T, int Mc) {
    constexpr int NQ = 8 * R;
    constexpr int MP = 64 * R;
    const int TS = T + 2;
    extern __shared__ float smem[];
    LdsHead hd(smem, T);
    float *col = hd.rest;            // [2][MP]
    float *sm_main = col + 2 * MP;   // [Mc][T]
    float *sm_leaf = sm_main + (TAB_LDS ? Mc * T : 0);
    float *sm_S = sm_leaf + (TAB_LDS ? Mc * T : 0);  // [Mc][TS]
    float *sm_F0 = sm_S + (TAB_LDS ? Mc * TS : 0);
    float *sm_F1 = sm_F0 + (TAB_LDS ? Mc * TS : 0);

    const int tid = threadIdx.x, j = tid & 7, g8 = (tid >> 3) & 7;
    const int p = wave_block(tid >> 6);
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *lk = links + (size_t)b * L * 2 * L;
    float *Sb = S + (size_t)b * Mc * TS;
    AuxView av(aux, b, Mc, T);

    if (!lengths_ok(m, n, L, T)) {  // out of contract: poison the log-likelihood, touch nothing else
        for (int i = tid; i < Mc * TS; i += NTR) Sb[i] = (i == 0) ? __builtin_nanf("") : NEG_INF_F;
        return;
    }
    const int mc = m / 2;  // active main-chain nodes: a_id < mc

    // link slabs -> registers; the loads are unconditional (clamped addresses) so that they are all in flight together
    float A0[R][NQ], A1[R][NQ];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a_id = 64 * r + 8 * p + g8;
        const size_t row = (size_t)(2 * min(a_id, Mc - 1) + 1) * 2;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int c = 2 * min(j + 8 * q, Mc - 1) + 1;
            A0[r][q] = lk[(row + 0) * L + c];
            A1[r][q] = lk[(row + 1) * L + c];
        }
    }
    const float base_cell = sanitize(mt[(size_t)(m - 1) * T + (n - 1)]);  // pcfg_loss.cu:142-147
    if (TAB_LDS) {
        for (int i = tid; i < Mc * T; i += NTR) {
            const int a_id = i / T, s = i - a_id * T;
            const float vm = mt[(size_t)(2 * a_id + 1) * T + s], vl = mt[(size_t)(2 * a_id) * T + s];
            const bool ok = a_id < mc && s < n;
            sm_main[i] = ok ? to_b2(vm) : NEG_INF_F;
            sm_leaf[i] = (ok && a_id >= 1) ? to_b2(vl) : NEG_INF_F;
        }
        for (int i = tid; i < Mc * TS; i += NTR) {
            sm_S[i] = (i == (mc - 1) * TS + (n - 1)) ? base_cell * LOG2E_F : NEG_INF_F;
            sm_F0[i] = NEG_INF_F;
            sm_F1[i] = NEG_INF_F;
        }
    } else {
        // cells of S and R the sweep never writes: rows beyond the sentence, columns from n-1 on (except the base cell)
        for (int i = tid; i < Mc * TS; i += NTR) {
            const int a_id = i / TS, s = i - a_id * TS;
            if (a_id >= mc || s >= n - 1) {
                const bool is_base = (a_id == mc - 1 && s == n - 1);
                Sb[i] = is_base ? base_cell : NEG_INF_F;
                av.SR[i] = is_base ? base_cell * LOG2E_F : NEG_INF_F;
            }
        }
    }
    for (int i = tid; i < MP; i += NTR) col[((n - 1) & 1) * MP + i] = (i == mc - 1) ? base_cell * LOG2E_F : NEG_INF_F;
    for (int i = tid; i < TS + 2; i += NTR) {
        hd.D[i] = 0.f;
        if (i < TS) hd.O[i] = 0.0;
    }
    if (tid < 16) hd.slots[tid] = base_cell * LOG2E_F;  // maximum of column n-1
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a_id = 64 * r + 8 * p + g8;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int c_id = j + 8 * q;
            const bool ok = a_id < mc && c_id < mc && c_id >= a_id;
            A0[r][q] = ok ? to_b2(A0[r][q]) : NEG_INF_F;
            A1[r][q] = (ok && a_id >= 1) ? to_b2(A1[r][q]) : NEG_INF_F;
        }
    }
    __syncthreads();
    FwdSweepArgs sa{col, sm_main, sm_leaf, sm_S, sm_F0, sm_F1, mt, Sb, av.F0, av.F1, av.SR, hd.slots, hd.D, hd.O, base_cell * LOG2E_F, n, mc, Mc, T, j, g8};
    switch (p) {  // wave-uniform: every wave runs the sweep specialised for its node block
        case 0: fwd_sweep<R, TAB_LDS, 0>(A0, A1, sa); break;
        case 1: fwd_sweep<R, TAB_LDS, 1>(A0, A1, sa); break;
        case 2: fwd_sweep<R, TAB_LDS, 2>(A0, A1, sa); break;
        case 3: fwd_sweep<R, TAB_LDS, 3>(A0, A1, sa); break;
        case 4: fwd_sweep<R, TAB_LDS, 4>(A0, A1, sa); break;
        case 5: fwd_sweep<R, TAB_LDS, 5>(A0, A1, sa); break;
        case 6: fwd_sweep<R, TAB_LDS, 6>(A0, A1, sa); break;
        default: fwd_sweep<R, TAB_LDS, 7>(A0, A1, sa); break;
    }
    if (TAB_LDS) {
        for (int i = tid; i < Mc * TS; i += NTR) {
            const int t = i - (i / TS) * TS;
            const float r2 = sm_S[i];
            Sb[i] = (float)(((double)r2 + hd.O[t]) * LN2_D);
            av.SR[i] = r2;
            av.F0[i] = sm_F0[i];
            av.F1[i] = sm_F1[i];
        }
    }
    for (int i = tid; i < TS + 2; i += NTR) {
        av.D[i] = hd.D[i];
        if (i < TS) av.O[i] = hd.O[i];
    }
}

template <int R, bool TAB_LDS>
__global__ __launch_bounds__(NTR) void inside_fwd_ml1_kernel(const float *__restrict__ match_all, const float *__restrict__ links,
                                                            const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                            float *__restrict__ S, float *__restrict__ aux, int L, int T, int Mc) {
    inside_fwd_ml1_body<R, TAB_LDS>(blockIdx.x, match_all, links, out_len, tgt_len, S, aux, L, T, Mc);
}

struct BwdSweepArgs {
    float *w0, *w1, *sm_S, *sm_B, *sm_main, *sm_leaf;
    const float *mt, *gSR;
    float *gBETA;
    const float *sm_D;
    float beta00;
    int n, mc, Mc, T, j, g8;
};

// The outside sweep of one wave, specialised on its node block P: only the chunks q <= 8r + P can hold parents a <= c.
template <int R, bool TAB_LDS, int P>
__device__ __forceinline__ void bwd_sweep(const float (&A0)[R][8 * R], const float (&A1)[R][8 * R], float (&G0)[R][8 * R],
                                          float (&G1)[R][8 * R], const BwdSweepArgs &x) {
    constexpr int NQ = 8 * R;
    constexpr int MP = 64 * R;
    const int T = x.T, TS = x.T + 2, j = x.j;
    float bprev[R];
#pragma unroll
    for (int r = 0; r < R; r++) bprev[r] = (64 * r + 8 * P + x.g8 == 0) ? x.beta00 : NEG_INF_F;
    for (int t = 1; t <= x.n - 1; t++) {
        const float *c0 = x.w0 + (t & 1) * MP, *c1 = x.w1 + (t & 1) * MP;
        float *n0 = x.w0 + ((t + 1) & 1) * MP, *n1 = x.w1 + ((t + 1) & 1) * MP;
        const float d_next = x.sm_D[t + 1], d_both = d_next + x.sm_D[t];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int c_id = 64 * r + 8 * P + x.g8;
            const int q_end = 8 * r + P + 1;  // chunks beyond hold only parents a > c
            const bool live = c_id < x.mc;
            const int ci = live ? c_id : 0;
            float u0[NQ], u1[NQ];
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q < q_end) {
                    u0[q] = c0[j + 8 * q];
                    u1[q] = c1[j + 8 * q];
                }
            }
            float sct, mc_t, ml_p;
            if (TAB_LDS) {
                sct = x.sm_S[ci * TS + t];
                mc_t = x.sm_main[ci * T + t];
                ml_p = x.sm_leaf[ci * T + t - 1];
            } else {
                sct = x.gSR[(size_t)ci * TS + t];
                mc_t = to_b2(x.mt[(size_t)(2 * ci + 1) * T + t]);
                const float xl = x.mt[(size_t)(2 * ci) * T + t - 1];
                ml_p = ci >= 1 ? to_b2(xl) : NEG_INF_F;
            }
            if (!live) {
                sct = NEG_INF_F;
                mc_t = NEG_INF_F;
                ml_p = NEG_INF_F;
            }
            float v0[NQ], v1[NQ];
            float mx = NEG_INF_F;
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q < q_end) {
                    v0[q] = A0[r][q] + u0[q];
                    v1[q] = A1[r][q] + u1[q];
                    mx = fmaxf(mx, fmaxf(v0[q], v1[q]));
                }
            }
            mx = row8_max(mx);
            const float mxs = (mx == NEG_INF_F) ? 0.f : mx;
            const float scale = (mx == NEG_INF_F || sct == NEG_INF_F) ? 0.f : ex2(mxs + sct);
            float sum = 0.f;
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q < q_end) {
                    const float e0 = ex2(v0[q] - mxs), e1 = ex2(v1[q] - mxs);
                    sum += e0 + e1;
                    G0[r][q] = __builtin_fmaf(e0, scale, G0[r][q]);
                    G1[r][q] = __builtin_fmaf(e1, scale, G1[r][q]);
                }
            }
            sum = row8_sum(sum);
            const float beta = (mx == NEG_INF_F || !live) ? NEG_INF_F : mx + lg2(sum);
            // outside weights this node offers to its children at the next two positions
            const float nw0 = (mc_t + beta) - d_next;
            const float nw1 = ((ml_p + mc_t) + bprev[r]) - d_both;
            bprev[r] = beta;
            if (j == 0) {
                n0[c_id] = nw0;
                n1[c_id] = nw1;
                if (live) {
                    if (TAB_LDS) x.sm_B[c_id * TS + t] = beta;
                    else x.gBETA[(size_t)c_id * TS + t] = beta;
                }
            }
        }
        lds_barrier();
    }
}

// Backward: outside sweep t = 1 .. n-1 (one 8-lane group per child node c, lanes strided over parents a <= c), rule
// posteriors accumulated in registers, then the element-wise emission epilogue.
// Dynamic LDS: head (see LdsHead), w0[2][MP], w1[2][MP]; with TAB_LDS also R, F0h, F1h, Bh [Mc][T+2] and the emissions of
// main nodes and leaves [Mc][T], all base 2: sweep and epilogue then read no global memory.
template <int R, bool TAB_LDS>
__global__ __launch_bounds__(NTR) void inside_bwd_ml1_kernel(const float *__restrict__ grad_out, const float *__restrict__ S,
                                                            float *__restrict__ aux, const float *__restrict__ match_all,
                                                            const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                            const int64_t *__restrict__ tgt_len, float *__restrict__ mgrad,
                                                            float *__restrict__ lgrad, int L, int T, int Mc, Seed seed) {
    constexpr int NQ = 8 * R;
    constexpr int MP = 64 * R;
    const int TS = T + 2;
    extern __shared__ float smem[];
    LdsHead hd(smem, T);
    float *w0 = hd.rest;         // [2][MP]
    float *w1 = w0 + 2 * MP;      // [2][MP]
    float *sm_S = w0 + 4 * MP;    // [Mc][TS]   (TAB_LDS)
    float *sm_F0 = sm_S + (TAB_LDS ? Mc * TS : 0);
    float *sm_F1 = sm_F0 + (TAB_LDS ? Mc * TS : 0);
    float *sm_B = sm_F1 + (TAB_LDS ? Mc * TS : 0);
    float *sm_main = sm_B + (TAB_LDS ? Mc * TS : 0);  // [Mc][T]
    float *sm_leaf = sm_main + (TAB_LDS ? Mc * T : 0);

    const int b = blockIdx.x, tid = threadIdx.x, j = tid & 7, g8 = (tid >> 3) & 7;
    const int p = wave_block(tid >> 6);
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *lk = links + (size_t)b * L * 2 * L;
    const float *Sb = S + (size_t)b * Mc * TS;
    float *mg = mgrad + (size_t)b * L * T;
    float *lg = lgrad + (size_t)b * L * 2 * L;
    AuxView av(aux, b, Mc, T);

    const float ll = Sb[0];
    const bool valid = lengths_ok(m, n, L, T) && (ll == ll) && (fabsf(ll) != __builtin_huge_valf());
    if (!valid) {  // invalid sentence: all-zero gradients (nat_pcfg_loss.py:123-133 zeroes its loss as well)
        for (int i = tid; i < L * T; i += NTR) mg[i] = 0.f;
        for (int i = tid; i < L * 2 * L; i += NTR) lg[i] = 0.f;
        return;
    }
    const int mc = m / 2;
    // a null grad_output selects the criterion's own weights: -factor/(n_b * norm_B), see Seed
    const float g = seed_weight(grad_out, b, n, seed);

    // links_grad is zero outside the cells the register accumulators own (written at the very end, after the barriers of
    // the sweep have ordered them behind this fill): clear the whole slab now, while the loads below are in flight
    {
        const int total = L * 2 * L;
        if ((total & 3) == 0 && (reinterpret_cast<uintptr_t>(lg) & 15) == 0) {
            float4 *lg4 = reinterpret_cast<float4 *>(lg);
            for (int i = tid; i < total / 4; i += NTR) lg4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (int i = tid; i < total; i += NTR) lg[i] = 0.f;
        }
    }
    // transposed link slabs: this thread's group owns child c, its lanes the parents a <= c; unconditional loads
    float A0[R][NQ], A1[R][NQ], G0[R][NQ], G1[R][NQ];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = 2 * min(64 * r + 8 * p + g8, Mc - 1) + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const size_t row = (size_t)(2 * min(j + 8 * q, Mc - 1) + 1) * 2;
            A0[r][q] = lk[(row + 0) * L + c];
            A1[r][q] = lk[(row + 1) * L + c];
            G0[r][q] = 0.f;
            G1[r][q] = 0.f;
        }
    }
    if (TAB_LDS) {
        for (int i = tid; i < Mc * T; i += NTR) {
            const int a_id = i / T, s = i - a_id * T;
            const float vm = mt[(size_t)(2 * a_id + 1) * T + s], vl = mt[(size_t)(2 * a_id) * T + s];
            const bool ok = a_id < mc && s < n;
            sm_main[i] = ok ? to_b2(vm) : NEG_INF_F;
            sm_leaf[i] = (ok && a_id >= 1) ? to_b2(vl) : NEG_INF_F;
        }
        for (int i = tid; i < Mc * TS; i += NTR) {
            sm_S[i] = av.SR[i];
            sm_F0[i] = av.F0[i];
            sm_F1[i] = av.F1[i];
            sm_B[i] = NEG_INF_F;
        }
    }
    for (int i = tid; i < TS + 2; i += NTR) hd.D[i] = av.D[i];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c_id = 64 * r + 8 * p + g8;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int a_id = j + 8 * q;
            const bool ok = a_id < mc && c_id < mc && a_id <= c_id;
            A0[r][q] = ok ? to_b2(A0[r][q]) : NEG_INF_F;
            A1[r][q] = (ok && a_id >= 1) ? to_b2(A1[r][q]) : NEG_INF_F;
        }
    }
    auto match_main = [&](int a_id, int s) -> float {
        if (TAB_LDS) return sm_main[a_id * T + s];
        return to_b2(mt[(size_t)(2 * a_id + 1) * T + s]);
    };
    auto match_leaf = [&](int a_id, int s) -> float {
        if (TAB_LDS) return sm_leaf[a_id * T + s];
        const float x = mt[(size_t)(2 * a_id) * T + s];
        return a_id >= 1 ? to_b2(x) : NEG_INF_F;
    };
    auto f0_at = [&](int a_id, int s) -> float { return TAB_LDS ? sm_F0[a_id * TS + s] : av.F0[(size_t)a_id * TS + s]; };
    auto f1_at = [&](int a_id, int s) -> float { return TAB_LDS ? sm_F1[a_id * TS + s] : av.F1[(size_t)a_id * TS + s]; };
    auto beta_at = [&](int a_id, int s) -> float { return TAB_LDS ? sm_B[a_id * TS + s] : av.BETA[(size_t)a_id * TS + s]; };

    const float beta00 = -av.SR[0];  // outside score of (root, 0), relative to the offset of column 0
    for (int i = tid; i < MP; i += NTR) {
        w0[1 * MP + i] = NEG_INF_F;
        w1[1 * MP + i] = NEG_INF_F;
    }
    if (!TAB_LDS)
        for (int i = tid; i < mc; i += NTR) av.BETA[(size_t)i * TS] = (i == 0) ? beta00 : NEG_INF_F;
    __syncthreads();
    if (tid == 0) {
        w0[1 * MP + 0] = (match_main(0, 0) + beta00) - hd.D[1];
        if (TAB_LDS) sm_B[0] = beta00;
    }
    __syncthreads();
    BwdSweepArgs sa{w0, w1, sm_S, sm_B, sm_main, sm_leaf, mt, av.SR, av.BETA, hd.D, beta00, n, mc, Mc, T, j, g8};
    switch (p) {  // wave-uniform
        case 0: bwd_sweep<R, TAB_LDS, 0>(A0, A1, G0, G1, sa); break;
        case 1: bwd_sweep<R, TAB_LDS, 1>(A0, A1, G0, G1, sa); break;
        case 2: bwd_sweep<R, TAB_LDS, 2>(A0, A1, G0, G1, sa); break;
        case 3: bwd_sweep<R, TAB_LDS, 3>(A0, A1, G0, G1, sa); break;
        case 4: bwd_sweep<R, TAB_LDS, 4>(A0, A1, G0, G1, sa); break;
        case 5: bwd_sweep<R, TAB_LDS, 5>(A0, A1, G0, G1, sa); break;
        case 6: bwd_sweep<R, TAB_LDS, 6>(A0, A1, G0, G1, sa); break;
        default: bwd_sweep<R, TAB_LDS, 7>(A0, A1, G0, G1, sa); break;
    }
    __syncthreads();  // BETA written by the group leaders is read by every thread below

    // rule posteriors -> links_grad (pcfg_loss_backward.cu:512-531); everything else in the slab is zero
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c_id = 64 * r + 8 * p + g8, c = 2 * c_id + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int a_id = j + 8 * q, a = 2 * a_id + 1;
            if (a_id < Mc && c_id < Mc && a_id <= c_id) {
                lg[((size_t)a * 2 + 0) * L + c] = g * G0[r][q];
                lg[((size_t)a * 2 + 1) * L + c] = g * G1[r][q];
            }
        }
    }
    // emission posteriors -> match_all_grad (pcfg_loss_backward.cu:348-382, 429-433)
    for (int i = tid; i < L * T; i += NTR) {
        const int x = i / T, s = i - x * T;
        float out = 0.f;
        if (x >= 1 && x < m && s < n) {
            const int a_id = x >> 1;
            if (x & 1) {
                const float bs = beta_at(a_id, s);
                const float mas = match_main(a_id, s);
                if (s + 1 <= n - 1) out += ex2(bs + mas + f0_at(a_id, s + 1));  // a emits s with the null left child
                if (s >= 1 && s + 1 <= n - 1 && a_id >= 1)                      // a emits s after its leaf emitted s-1
                    out += ex2(beta_at(a_id, s - 1) + match_leaf(a_id, s - 1) + mas + (f1_at(a_id, s + 1) - hd.D[s]));
                if (a_id == mc - 1 && s == n - 1) out += ex2(bs + mas);        // base cell
            } else if (a_id >= 1 && a_id < mc && s + 2 <= n - 1) {             // leaf of parent a = x+1
                out += ex2(beta_at(a_id, s) + match_leaf(a_id, s) + match_main(a_id, s + 1) + (f1_at(a_id, s + 2) - hd.D[s + 1]));
            }
            if (!(out == out)) out = 0.f;
        }
        mg[i] = g * out;
    }
}

// Forward and backward in one launch, one workgroup per sentence (the single call's path where the paired sweeps further
// down do not apply: more than 128 nodes, or tables beyond their LDS budget but within this kernel's): the
// tables the backward needs (S, F0, F1, emissions) never leave LDS, only S is also written to global memory in the
// reference's layout.  Dynamic LDS: head (see LdsHead), w0[2][MP] (doubles as the forward's columns), w1[2][MP],
// R/F0h/F1h/Bh [Mc][T+2], emissions of main nodes and leaves [Mc][T].
template <int R>
__global__ __launch_bounds__(NTR) void inside_fused_ml1_kernel(const float *__restrict__ grad_out, const float *__restrict__ match_all,
                                                              const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                              const int64_t *__restrict__ tgt_len, float *__restrict__ S,
                                                              float *__restrict__ mgrad, float *__restrict__ lgrad, int L, int T,
                                                              int Mc, Seed seed) {
    constexpr int NQ = 8 * R;
    constexpr int MP = 64 * R;
    const int TS = T + 2;
    extern __shared__ float smem[];
    LdsHead hd(smem, T);
    float *w0 = hd.rest;         // [2][MP]
    float *w1 = w0 + 2 * MP;      // [2][MP]
    float *sm_S = w0 + 4 * MP;    // [Mc][TS]
    float *sm_F0 = sm_S + Mc * TS;
    float *sm_F1 = sm_F0 + Mc * TS;
    float *sm_B = sm_F1 + Mc * TS;
    float *sm_main = sm_B + Mc * TS;  // [Mc][T]
    float *sm_leaf = sm_main + Mc * T;

    const int b = blockIdx.x, tid = threadIdx.x, j = tid & 7, g8 = (tid >> 3) & 7;
    const int p = wave_block(tid >> 6);
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *lk = links + (size_t)b * L * 2 * L;
    float *Sb = S + (size_t)b * Mc * TS;
    float *mg = mgrad + (size_t)b * L * T;
    float *lg = lgrad + (size_t)b * L * 2 * L;

    {   // links_grad: everything outside the accumulator-owned cells is zero (see inside_bwd_ml1_kernel)
        const int total = L * 2 * L;
        if ((total & 3) == 0 && (reinterpret_cast<uintptr_t>(lg) & 15) == 0) {
            float4 *lg4 = reinterpret_cast<float4 *>(lg);
            for (int i = tid; i < total / 4; i += NTR) lg4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (int i = tid; i < total; i += NTR) lg[i] = 0.f;
        }
    }
    if (!lengths_ok(m, n, L, T)) {  // out of contract: poisoned log-likelihood, zero gradients
        for (int i = tid; i < Mc * TS; i += NTR) Sb[i] = (i == 0) ? __builtin_nanf("") : NEG_INF_F;
        for (int i = tid; i < L * T; i += NTR) mg[i] = 0.f;
        return;
    }
    const int mc = m / 2;
    const float g = seed_weight(grad_out, b, n, seed);

    // ---- forward
    float A0[R][NQ], A1[R][NQ];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const size_t row = (size_t)(2 * min(64 * r + 8 * p + g8, Mc - 1) + 1) * 2;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int c = 2 * min(j + 8 * q, Mc - 1) + 1;
            A0[r][q] = lk[(row + 0) * L + c];
            A1[r][q] = lk[(row + 1) * L + c];
        }
    }
    const float base_cell = sanitize(mt[(size_t)(m - 1) * T + (n - 1)]);
    for (int i = tid; i < Mc * T; i += NTR) {
        const int a_id = i / T, s = i - a_id * T;
        const float vm = mt[(size_t)(2 * a_id + 1) * T + s], vl = mt[(size_t)(2 * a_id) * T + s];
        const bool ok = a_id < mc && s < n;
        sm_main[i] = ok ? to_b2(vm) : NEG_INF_F;
        sm_leaf[i] = (ok && a_id >= 1) ? to_b2(vl) : NEG_INF_F;
    }
    for (int i = tid; i < Mc * TS; i += NTR) {
        sm_S[i] = (i == (mc - 1) * TS + (n - 1)) ? base_cell * LOG2E_F : NEG_INF_F;
        sm_F0[i] = NEG_INF_F;
        sm_F1[i] = NEG_INF_F;
        sm_B[i] = NEG_INF_F;
    }
    for (int i = tid; i < MP; i += NTR) w0[((n - 1) & 1) * MP + i] = (i == mc - 1) ? base_cell * LOG2E_F : NEG_INF_F;
    for (int i = tid; i < TS + 2; i += NTR) {
        hd.D[i] = 0.f;
        if (i < TS) hd.O[i] = 0.0;
    }
    if (tid < 16) hd.slots[tid] = base_cell * LOG2E_F;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a_id = 64 * r + 8 * p + g8;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int c_id = j + 8 * q;
            const bool ok = a_id < mc && c_id < mc && c_id >= a_id;
            A0[r][q] = ok ? to_b2(A0[r][q]) : NEG_INF_F;
            A1[r][q] = (ok && a_id >= 1) ? to_b2(A1[r][q]) : NEG_INF_F;
        }
    }
    __syncthreads();
    {
        FwdSweepArgs sa{w0, sm_main, sm_leaf, sm_S, sm_F0, sm_F1, mt, Sb, nullptr, nullptr, nullptr, hd.slots, hd.D, hd.O, base_cell * LOG2E_F, n, mc, Mc, T, j, g8};
        switch (p) {
            case 0: fwd_sweep<R, true, 0>(A0, A1, sa); break;
            case 1: fwd_sweep<R, true, 1>(A0, A1, sa); break;
            case 2: fwd_sweep<R, true, 2>(A0, A1, sa); break;
            case 3: fwd_sweep<R, true, 3>(A0, A1, sa); break;
            case 4: fwd_sweep<R, true, 4>(A0, A1, sa); break;
            case 5: fwd_sweep<R, true, 5>(A0, A1, sa); break;
            case 6: fwd_sweep<R, true, 6>(A0, A1, sa); break;
            default: fwd_sweep<R, true, 7>(A0, A1, sa); break;
        }
    }
    // ---- backward: transposed slabs are requested first, S goes out to global memory while they travel
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = 2 * min(64 * r + 8 * p + g8, Mc - 1) + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const size_t row = (size_t)(2 * min(j + 8 * q, Mc - 1) + 1) * 2;
            A0[r][q] = lk[(row + 0) * L + c];
            A1[r][q] = lk[(row + 1) * L + c];
        }
    }
    for (int i = tid; i < Mc * TS; i += NTR) {
        const int t = i - (i / TS) * TS;
        Sb[i] = (float)(((double)sm_S[i] + hd.O[t]) * LN2_D);
    }
    const float ll2 = sm_S[0];  // base 2, relative to the offset of column 0
    const bool valid = (ll2 == ll2) && (fabsf(ll2) != __builtin_huge_valf());
    if (!valid) {  // workgroup-uniform
        for (int i = tid; i < L * T; i += NTR) mg[i] = 0.f;
        return;
    }
    float G0[R][NQ], G1[R][NQ];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c_id = 64 * r + 8 * p + g8;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int a_id = j + 8 * q;
            const bool ok = a_id < mc && c_id < mc && a_id <= c_id;
            A0[r][q] = ok ? to_b2(A0[r][q]) : NEG_INF_F;
            A1[r][q] = (ok && a_id >= 1) ? to_b2(A1[r][q]) : NEG_INF_F;
            G0[r][q] = 0.f;
            G1[r][q] = 0.f;
        }
    }
    const float beta00 = -ll2;
    for (int i = tid; i < MP; i += NTR) {
        w0[1 * MP + i] = (i == 0) ? (sm_main[0] + beta00) - hd.D[1] : NEG_INF_F;
        w1[1 * MP + i] = NEG_INF_F;
    }
    if (tid == 0) sm_B[0] = beta00;
    __syncthreads();
    {
        BwdSweepArgs sa{w0, w1, sm_S, sm_B, sm_main, sm_leaf, mt, nullptr, nullptr, hd.D, beta00, n, mc, Mc, T, j, g8};
        switch (p) {
            case 0: bwd_sweep<R, true, 0>(A0, A1, G0, G1, sa); break;
            case 1: bwd_sweep<R, true, 1>(A0, A1, G0, G1, sa); break;
            case 2: bwd_sweep<R, true, 2>(A0, A1, G0, G1, sa); break;
            case 3: bwd_sweep<R, true, 3>(A0, A1, G0, G1, sa); break;
            case 4: bwd_sweep<R, true, 4>(A0, A1, G0, G1, sa); break;
            case 5: bwd_sweep<R, true, 5>(A0, A1, G0, G1, sa); break;
            case 6: bwd_sweep<R, true, 6>(A0, A1, G0, G1, sa); break;
            default: bwd_sweep<R, true, 7>(A0, A1, G0, G1, sa); break;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c_id = 64 * r + 8 * p + g8, c = 2 * c_id + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const int a_id = j + 8 * q, a = 2 * a_id + 1;
            if (a_id < Mc && c_id < Mc && a_id <= c_id) {
                lg[((size_t)a * 2 + 0) * L + c] = g * G0[r][q];
                lg[((size_t)a * 2 + 1) * L + c] = g * G1[r][q];
            }
        }
    }
    for (int i = tid; i < L * T; i += NTR) {
        const int x = i / T, s = i - x * T;
        float out = 0.f;
        if (x >= 1 && x < m && s < n) {
            const int a_id = x >> 1;
            if (x & 1) {
                const float bs = sm_B[a_id * TS + s];
                const float mas = sm_main[a_id * T + s];
                if (s + 1 <= n - 1) out += ex2(bs + mas + sm_F0[a_id * TS + s + 1]);
                if (s >= 1 && s + 1 <= n - 1 && a_id >= 1)
                    out += ex2(sm_B[a_id * TS + s - 1] + sm_leaf[a_id * T + s - 1] + mas + (sm_F1[a_id * TS + s + 1] - hd.D[s]));
                if (a_id == mc - 1 && s == n - 1) out += ex2(bs + mas);
            } else if (a_id >= 1 && a_id < mc && s + 2 <= n - 1) {
                out += ex2(sm_B[a_id * TS + s] + sm_leaf[a_id * T + s] + sm_main[a_id * T + s + 1] +
                           (sm_F1[a_id * TS + s + 2] - hd.D[s + 1]));
            }
            if (!(out == out)) out = 0.f;
        }
        mg[i] = g * out;
    }
}

// ------------------------------------------------------------------------------------------------------------
// Forward and outside sweep side by side (graphs of up to 130 nodes).  The outside recurrence (see the top of inside.hip)
// only needs the links, the emissions and its own earlier columns - the inside table enters the posteriors, not the sweep
// - so the two sweeps of a sentence are independent chains.  One workgroup already saturates the instruction issue of
// its compute unit with one sweep, so they run as two workgroups: inside_pair_ml1_kernel launches 2B of them, the even
// ones do what inside_fwd_ml1_kernel does, the odd ones the outside sweep, which halves the sequential part of the pass;
// inside_combine_ml1_kernel then turns the tables into posteriors, in parallel over the cells.
//
// The outside sweep cannot use the forward's column offsets (they are being produced at the other end of the sentence),
// so it keeps offsets of its own: beta[root][0] = 0, W_t columns relative to P_t = E_1 + .. + E_t with the shift E_{t+1}
// chosen as the maximum of the relative beta column t-1.  Posteriors then take one correction per column,
//   corr_t  = P_t     + O_t - ll      (rule a -> c at column t; emission with the null left child; base cell)
//   corr1_t = P_{t-1} + O_t - ll      (emissions that go through the local leaf),
// computed in double from the two offset sequences.
// ------------------------------------------------------------------------------------------------------------
struct OutsideFreeArgs {
    float *w0, *w1;                // rotating columns [2][64]
    float *sm_B, *sm_W0, *sm_W1;   // tables [Mc][T+2]
    const float *sm_main, *sm_leaf;
    float *slots;                  // [2][8] per-wave maxima of the relative beta columns
    float *sm_E;                   // [T+4] shifts
    double *sm_P;                  // [T+4] offsets
    int n, mc, T, j, g8, wave;
};

template <int P>
__device__ __forceinline__ void outside_sweep_free(const float (&A0)[1][8], const float (&A1)[1][8], const OutsideFreeArgs &x) {
    constexpr int NQ = 8, MP = 64;
    const int T = x.T, TS = x.T + 2, j = x.j;
    const int c_id = 8 * P + x.g8;
    const int q_end = P + 1;  // chunks beyond hold only parents a > c
    const bool live = c_id < x.mc;
    const int ci = live ? c_id : 0;
    float bprev = live ? x.sm_B[ci * TS] : NEG_INF_F;  // relative beta of column t-1 (beta[root][0] = 0)
    float e_cur = x.sm_E[1];                           // E_t
    double Pt = x.sm_P[1];                             // P_t
    for (int t = 1; t <= x.n - 1; t++) {
        const float *c0 = x.w0 + (t & 1) * MP, *c1 = x.w1 + (t & 1) * MP;
        float *n0 = x.w0 + ((t + 1) & 1) * MP, *n1 = x.w1 + ((t + 1) & 1) * MP;
        float u0[NQ], u1[NQ];
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q < q_end) {
                u0[q] = c0[j + 8 * q];
                u1[q] = c1[j + 8 * q];
            }
        }
        // shift of the next column: the maximum of the relative beta column t-1, published one step ago
        const float Dm = max8(x.slots + ((t - 1) & 1) * 8);
        const float e_next = (Dm == NEG_INF_F) ? 0.f : Dm;
        const double P_next = Pt + (double)e_next;
        if (x.wave == 0 && j == 0 && x.g8 == 0) {
            x.sm_E[t + 1] = e_next;
            x.sm_P[t + 1] = P_next;
        }
        float mc_t = x.sm_main[ci * T + t], ml_p = x.sm_leaf[ci * T + t - 1];
        if (!live) {
            mc_t = NEG_INF_F;
            ml_p = NEG_INF_F;
        }
        float v0[NQ], v1[NQ];
        float mx = NEG_INF_F;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q < q_end) {
                v0[q] = A0[0][q] + u0[q];
                v1[q] = A1[0][q] + u1[q];
                mx = fmaxf(mx, fmaxf(v0[q], v1[q]));
            }
        }
        mx = row8_max(mx);
        const float mxs = (mx == NEG_INF_F) ? 0.f : mx;
        float sum = 0.f;
#pragma unroll
        for (int q = 0; q < NQ; q++)
            if (q < q_end) sum += ex2(v0[q] - mxs) + ex2(v1[q] - mxs);
        sum = row8_sum(sum);
        const float beta = (mx == NEG_INF_F || !live) ? NEG_INF_F : mx + lg2(sum);
        // outside weights this node offers to its children at the next two positions
        const float nw0 = (mc_t + beta) - e_next;
        const float nw1 = ((ml_p + mc_t) + bprev) - (e_next + e_cur);
        bprev = beta;
        const float wm = wave_max_of_groups(beta + 0.f);
        if ((threadIdx.x & 63) == 0) x.slots[(t & 1) * 8 + x.wave] = wm;
        if (j == 0) {
            n0[c_id] = nw0;
            n1[c_id] = nw1;
            if (live) {
                x.sm_B[c_id * TS + t] = beta;
                x.sm_W0[c_id * TS + t + 1] = nw0;
                x.sm_W1[c_id * TS + t + 1] = nw1;
            }
        }
        e_cur = e_next;
        Pt = P_next;
        lds_barrier();
    }
}

// Dynamic LDS of the outside role: P [T+4] (double), slots [16], E [T+4], w0 [2][64], w1 [2][64], Bh, W0h, W1h [Mc][T+2],
// emissions of main nodes and leaves [Mc][T].
__host__ __device__ inline size_t outside_role_bytes(int Mc, int T) {
    return (size_t)(T + 4) * sizeof(double) + ((size_t)16 + (T + 4) + 4 * 64 + (size_t)3 * Mc * (T + 2) + (size_t)2 * Mc * T) * sizeof(float);
}

__device__ __forceinline__ void inside_outside_ml1_body(const int b, const float *__restrict__ match_all,
                                                       const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                       const int64_t *__restrict__ tgt_len, float *__restrict__ aux, int L, int T,
                                                       int Mc) {
    constexpr int NQ = 8, MP = 64;
    const int TS = T + 2, TP = T + 4;
    extern __shared__ double smem_d[];
    double *sm_P = smem_d;                                    // [TP]
    float *slots = reinterpret_cast<float *>(sm_P + TP);     // [16]
    float *sm_E = slots + 16;                                 // [TP]
    float *w0 = sm_E + TP;                                    // [2][MP]
    float *w1 = w0 + 2 * MP;                                  // [2][MP]
    float *sm_B = w1 + 2 * MP;                                // [Mc][TS] each
    float *sm_W0 = sm_B + Mc * TS;
    float *sm_W1 = sm_W0 + Mc * TS;
    float *sm_main = sm_W1 + Mc * TS;                         // [Mc][T]
    float *sm_leaf = sm_main + Mc * T;

    const int tid = threadIdx.x, j = tid & 7, g8 = (tid >> 3) & 7;
    const int p = wave_block(tid >> 6);
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    if (!lengths_ok(m, n, L, T)) return;  // the forward role poisons the log-likelihood, the combine kernel writes zeros
    const int mc = m / 2;
    const float *mt = match_all + (size_t)b * L * T;
    const float *lk = links + (size_t)b * L * 2 * L;
    AuxView av(aux, b, Mc, T);

    // transposed link slabs: this thread's group owns child c, its lanes the parents a <= c; unconditional loads
    const int own = 8 * p + g8;
    float A0[1][NQ], A1[1][NQ];
    {
        const int c = 2 * min(own, Mc - 1) + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const size_t row = (size_t)(2 * min(j + 8 * q, Mc - 1) + 1) * 2;
            A0[0][q] = lk[(row + 0) * L + c];
            A1[0][q] = lk[(row + 1) * L + c];
        }
    }
    for (int i = tid; i < Mc * T; i += NTR) {
        const int a_id = i / T, s = i - a_id * T;
        const float vm = mt[(size_t)(2 * a_id + 1) * T + s], vl = mt[(size_t)(2 * a_id) * T + s];
        const bool ok = a_id < mc && s < n;
        sm_main[i] = ok ? to_b2(vm) : NEG_INF_F;
        sm_leaf[i] = (ok && a_id >= 1) ? to_b2(vl) : NEG_INF_F;
    }
    for (int i = tid; i < Mc * TS; i += NTR) {
        sm_B[i] = (i == 0) ? 0.f : NEG_INF_F;  // beta[root][0] = 0
        sm_W0[i] = NEG_INF_F;
        sm_W1[i] = NEG_INF_F;
    }
    for (int i = tid; i < 2 * MP; i += NTR) {
        w0[i] = NEG_INF_F;
        w1[i] = NEG_INF_F;
    }
    for (int i = tid; i < TP; i += NTR) {
        sm_E[i] = 0.f;
        sm_P[i] = 0.0;
    }
    if (tid < 16) slots[tid] = (tid < 8) ? 0.f : NEG_INF_F;  // maximum of the relative beta column 0
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        const int a_id = j + 8 * q;
        const bool ok = a_id < mc && own < mc && a_id <= own;
        A0[0][q] = ok ? to_b2(A0[0][q]) : NEG_INF_F;
        A1[0][q] = (ok && a_id >= 1) ? to_b2(A1[0][q]) : NEG_INF_F;
    }
    __syncthreads();
    if (tid == 0) {  // W_1 columns: the root offers match[root][0] to its null-left children
        const float w00 = sm_main[0];
        w0[1 * MP + 0] = w00;
        sm_W0[0 * TS + 1] = w00;
    }
    __syncthreads();
    {
        OutsideFreeArgs sa{w0, w1, sm_B, sm_W0, sm_W1, sm_main, sm_leaf, slots, sm_E, sm_P, n, mc, T, j, g8, (tid >> 6)};
        switch (p) {  // wave-uniform
            case 0: outside_sweep_free<0>(A0, A1, sa); break;
            case 1: outside_sweep_free<1>(A0, A1, sa); break;
            case 2: outside_sweep_free<2>(A0, A1, sa); break;
            case 3: outside_sweep_free<3>(A0, A1, sa); break;
            case 4: outside_sweep_free<4>(A0, A1, sa); break;
            case 5: outside_sweep_free<5>(A0, A1, sa); break;
            case 6: outside_sweep_free<6>(A0, A1, sa); break;
            default: outside_sweep_free<7>(A0, A1, sa); break;
        }
    }
    __syncthreads();
    for (int i = tid; i < Mc * TS; i += NTR) {
        av.BETA[i] = sm_B[i];
        av.W0[i] = sm_W0[i];
        av.W1[i] = sm_W1[i];
    }
    for (int i = tid; i < TP; i += NTR) {
        av.E[i] = sm_E[i];
        av.P[i] = sm_P[i];
    }
}

// Workgroups per sentence that zero the rows of its pad nodes (see PadFill) beside the sweeps.  One fill workgroup per
// compute unit on the units the sweeps leave free writes about 4.3 TB/s: beside the sweeps (29 us) the whole fill fits.
constexpr int PAD_WGS = 32;
// The fill rides along while the sweeps take up no more than three quarters of the compute units (192 of 256 on MI355X).
inline int pad_max_sweep_wgs() { return device_compute_units() * 3 / 4; }
constexpr size_t PAD_EXCLUSIVE_LDS = 84 * 1024;  // more than half of the 160 KB of a gfx950 compute unit

// Zeroes the bytes of rows [m_b, L) of sentence b - one contiguous span - as one of PAD_WGS workgroups: 16-byte
// streaming stores over the aligned body, byte stores over what is left at either end.
__device__ __forceinline__ void pad_fill_block(const PadFill pad, const int64_t *__restrict__ out_len, int b, int part, int L) {
    const int tid = threadIdx.x, NTF = blockDim.x;
    int64_t m = out_len[b];
    m = m < 0 ? 0 : (m > L ? L : m);
    unsigned char *begin = pad.base + ((int64_t)b * L + m) * pad.row_bytes;
    unsigned char *end = pad.base + ((int64_t)b + 1) * L * pad.row_bytes;
    if (begin >= end) return;
    unsigned char *body = reinterpret_cast<unsigned char *>((reinterpret_cast<uintptr_t>(begin) + 15) & ~(uintptr_t)15);
    unsigned char *body_end = reinterpret_cast<unsigned char *>(reinterpret_cast<uintptr_t>(end) & ~(uintptr_t)15);
    if (body >= body_end) {  // shorter than one aligned chunk
        if (part == 0)
            for (unsigned char *q = begin + tid; q < end; q += NTF) *q = 0;
        return;
    }
    if (part == 0) {
        if (begin + tid < body) begin[tid] = 0;
        if (body_end + tid < end) body_end[tid] = 0;
    }
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 *v = reinterpret_cast<u32x4 *>(body);
    const int64_t nv = (body_end - body) >> 4, per = (nv + PAD_WGS - 1) / PAD_WGS;
    const int64_t lo = per * part, hi = (lo + per < nv) ? lo + per : nv;
    u32x4 zero;
    zero.x = zero.y = zero.z = zero.w = 0;
    for (int64_t i = lo + tid; i < hi; i += NTF) __builtin_nontemporal_store(zero, v + i);
}

// 2*nsent workgroups: 2b runs the forward sweep of sentence b, 2b+1 its outside sweep; PAD_WGS*nsent more when
// there is a pad-fill task, which land on the compute units the sweeps leave free.
__global__ __launch_bounds__(NTR) void inside_pair_ml1_kernel(const float *__restrict__ match_all, const float *__restrict__ links,
                                                             const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                             float *__restrict__ S, float *__restrict__ aux, int L, int T, int Mc,
                                                             int nsent, PadFill pad) {
    if ((int)blockIdx.x >= 2 * nsent) {  // workgroup-uniform
        const int z = (int)blockIdx.x - 2 * nsent;
        pad_fill_block(pad, out_len, z / PAD_WGS, z % PAD_WGS, L);
        return;
    }
    const int b = blockIdx.x >> 1;
    if ((blockIdx.x & 1) == 0) inside_fwd_ml1_body<1, true>(b, match_all, links, out_len, tgt_len, S, aux, L, T, Mc);
    else inside_outside_ml1_body(b, match_all, links, out_len, tgt_len, aux, L, T, Mc);
}

// Posteriors from the tables of the two sweeps: grid (16, B), 256 threads.  Workgroup (q, b) owns the parents 4q .. 4q+3 of
// sentence b: it writes the rows 8q .. 8q+7 of the links_grad slab (zeros included) and a sixteenth of the match_all_grad
// cells.  One thread per (parent, child) pair sums both planes over the columns.
// Dynamic LDS: corr [T+4], R [Mc][T+2], W0h, W1h of the workgroup's parents [4][T+2].
__global__ __launch_bounds__(256) void inside_combine_ml1_kernel(const float *__restrict__ grad_out, const float *__restrict__ S,
                                                                float *__restrict__ aux, const float *__restrict__ match_all,
                                                                const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                                const int64_t *__restrict__ tgt_len, float *__restrict__ mgrad,
                                                                float *__restrict__ lgrad, int L, int T, int Mc, Seed seed,
                                                                LossTask loss) {
    // With a loss to form (the criterion's forward under autograd), the launch has one more row of workgroups, whose first
    // one reduces the log-likelihoods the sweeps left - beside the posteriors instead of in a launch of its own behind them.
    if (loss.out != nullptr && blockIdx.y == gridDim.y - 1) {  // workgroup-uniform
        if (blockIdx.x == 0) criterion_loss_block<256>(loss);
        return;
    }
    const int TS = T + 2, TP = T + 4;
    extern __shared__ float smem[];
    float *corr = smem;               // [TP]
    float *sm_R = corr + TP;          // [Mc][TS]
    float *sm_W0 = sm_R + Mc * TS;    // [4][TS]
    float *sm_W1 = sm_W0 + 4 * TS;    // [4][TS]
    const int part = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *lk = links + (size_t)b * L * 2 * L;
    float *mg = mgrad + (size_t)b * L * T;
    float *lg = lgrad + (size_t)b * L * 2 * L;
    AuxView av(aux, b, Mc, T);
    const int cells = L * T, cell0 = (int)((int64_t)cells * part / 16), cell1 = (int)((int64_t)cells * (part + 1) / 16);
    const int row0 = min(8 * part, L), row1 = min(8 * part + 8, L);
    for (int i = row0 * 2 * L + tid; i < row1 * 2 * L; i += 256) lg[i] = 0.f;

    // Everything this thread will read is requested here, before anything is used: no address depends on a loaded value
    // (indices are clamped, the lengths only decide later which values count), so the launch pays one trip to memory
    // instead of one per stage - which matters most while the pad fill beside it keeps the memory system busy.
    const float ll = S[(size_t)b * Mc * TS];
    // this thread's pair: parent 4*part + tid/64, child tid%64
    const int a_id = 4 * part + (tid >> 6), c_id = tid & 63;
    const size_t cell = ((size_t)(2 * min(a_id, Mc - 1) + 1) * 2) * L + 2 * min(c_id, Mc - 1) + 1;
    const float l0 = lk[cell], l1 = lk[cell + L];
    const double sr0 = (double)av.SR[0], o0 = av.O[0];
    const int tc = min(tid, TP - 1);
    const double p_t = av.P[tc], o_t = av.O[tc];
    constexpr int RV = 16;  // R table: up to 16 * 256 entries (64 nodes, T + 2 <= 64)
    float rv[RV];
#pragma unroll
    for (int k = 0; k < RV; k++) rv[k] = av.SR[min(k * 256 + tid, Mc * TS - 1)];
    const int wi = min(tid, 4 * TS - 1);
    const bool w_in = 4 * part + wi / TS < Mc;
    const size_t w_at = w_in ? (size_t)4 * part * TS + wi : 0;
    const float w0v = av.W0[w_at], w1v = av.W1[w_at];
    // the operands of this thread's first emission cell (clamped addresses; the cell's case picks the terms later)
    struct CellIn {
        double ps, os, ps1, os1;
        float bs, bs1, f0n, f1n, f1nn, mas, mprev, mnext;
    };
    auto load_cell = [&](int i) {
        CellIn c;
        const int x = i / T, s = i - x * T, e_id = x >> 1;
        const size_t o = (size_t)min(e_id, Mc - 1) * TS + s;
        c.ps = av.P[s];
        c.os = av.O[s];
        c.ps1 = av.P[max(s, 1) - 1];
        c.os1 = av.O[s + 1];
        c.bs = av.BETA[o];
        c.bs1 = av.BETA[max(o, (size_t)1) - 1];
        c.f0n = av.F0[o + 1];
        c.f1n = av.F1[o + 1];
        c.f1nn = av.F1[o + 2];
        c.mas = mt[i];
        c.mprev = mt[max(i - T - 1, 0)];            // (x-1, s-1): the leaf's emission before parent x
        c.mnext = mt[min(i + T + 1, L * T - 1)];    // (x+1, s+1): the parent's emission after leaf x
        return c;
    };
    const CellIn first = load_cell(min(cell0 + tid, cells - 1));

    const bool valid = lengths_ok(m, n, L, T) && (ll == ll) && (fabsf(ll) != __builtin_huge_valf());
    if (!valid) {  // invalid sentence: all-zero gradients (nat_pcfg_loss.py:123-133 zeroes its loss as well)
        for (int i = cell0 + tid; i < cell1; i += 256) mg[i] = 0.f;
        return;
    }
    const int mc = m / 2;
    // a null grad_output selects the criterion's own weights: -factor/(n_b * norm_B), see Seed
    const float g = seed_weight(grad_out, b, n, seed);
    const bool pair_ok = a_id < mc && c_id < mc && a_id <= c_id;
    const double ll_abs = sr0 + o0;
    if (tid <= n - 1) corr[tid] = (float)(p_t + o_t - ll_abs);
    for (int t = tid + 256; t <= n - 1; t += 256) corr[t] = (float)(av.P[t] + av.O[t] - ll_abs);
#pragma unroll
    for (int k = 0; k < RV; k++)
        if (k * 256 + tid < Mc * TS) sm_R[k * 256 + tid] = rv[k];
    for (int i = RV * 256 + tid; i < Mc * TS; i += 256) sm_R[i] = av.SR[i];
    if (tid < 4 * TS) {
        sm_W0[tid] = w_in ? w0v : NEG_INF_F;
        sm_W1[tid] = w_in ? w1v : NEG_INF_F;
    }
    for (int i = tid + 256; i < 4 * TS; i += 256) {
        const bool in = 4 * part + i / TS < Mc;
        sm_W0[i] = in ? av.W0[(size_t)4 * part * TS + i] : NEG_INF_F;
        sm_W1[i] = in ? av.W1[(size_t)4 * part * TS + i] : NEG_INF_F;
    }
    // emission posteriors -> match_all_grad (pcfg_loss_backward.cu:348-382, 429-433)
    for (int i = cell0 + tid; i < cell1; i += 256) {
        const CellIn c = (i == cell0 + tid) ? first : load_cell(i);
        const int x = i / T, s = i - x * T, e_id = x >> 1;
        const float mas = to_b2(c.mas), mprev = to_b2(c.mprev), mnext = to_b2(c.mnext);
        const float cs = (float)(c.ps + c.os - ll_abs), cs1 = (float)(c.ps1 + c.os - ll_abs), cs2 = (float)(c.ps + c.os1 - ll_abs);
        const bool in = x >= 1 && x < m && s < n, odd = x & 1;
        float out = 0.f;
        // a emits s with the null left child
        out += (in && odd && s + 1 <= n - 1) ? ex2((c.bs + mas + c.f0n) + cs) : 0.f;
        // a emits s after its leaf emitted s-1
        out += (in && odd && s >= 1 && s + 1 <= n - 1 && e_id >= 1) ? ex2((c.bs1 + mprev + mas + c.f1n) + cs1) : 0.f;
        // base cell
        out += (in && odd && e_id == mc - 1 && s == n - 1) ? ex2((c.bs + mas) + cs) : 0.f;
        // leaf of parent a = x+1
        out += (in && !odd && e_id >= 1 && e_id < mc && s + 2 <= n - 1) ? ex2((c.bs + mas + mnext + c.f1nn) + cs2) : 0.f;
        if (!(out == out)) out = 0.f;
        mg[i] = g * out;
    }
    __syncthreads();  // also orders the zero fill of the slab rows before the posteriors written below

    // rule posteriors -> links_grad (pcfg_loss_backward.cu:512-531): lg[a][k][c] = g * sum_t 2^(links + Wkh_t[a] + R_t[c] + corr_t)
    if (pair_ok) {
        const float A0 = to_b2(l0), A1 = (a_id >= 1) ? to_b2(l1) : NEG_INF_F;
        const float *w0r = sm_W0 + (tid >> 6) * TS, *w1r = sm_W1 + (tid >> 6) * TS, *rr = sm_R + c_id * TS;
        float acc0 = 0.f, acc1 = 0.f;
        for (int t = 1; t <= n - 1; t++) {
            const float rc = rr[t] + corr[t];
            acc0 += ex2((A0 + w0r[t]) + rc);
            acc1 += ex2((A1 + w1r[t]) + rc);
        }
        lg[cell] = g * ((acc0 == acc0) ? acc0 : 0.f);
        lg[cell + L] = g * ((acc1 == acc1) ? acc1 : 0.f);
    }
}

}  // namespace
}  // namespace pcfgnat
