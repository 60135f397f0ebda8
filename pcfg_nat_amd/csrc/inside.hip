// PCFG inside algorithm (loss forward), its exact backward, and the GLAT best-tree trace, for max_left = 1.
//
// Replaces the reference's pcfg_loss.cu (calculate_C_kernel :262-349, calculate_S_kernel :84-224),
// pcfg_loss_backward.cu (seven kernels, :28-603) and pcfg_best_tree.cu (:64-301).
//
// With max_left = 1 (every shipped configuration) main-chain node a = 2*a_id+1 has one local leaf a-1 and the
// recurrences collapse to
//   S[a][s] = LSE( match[a][s]                 + F0[a][s+1],      F0[a][t] = LSE_{c>=a} links[a][0][c] + S[c][t]
//                  match[a-1][s] + match[a][s+1] + F1[a][s+2] )     F1[a][t] = LSE_{c>=a} links[a][1][c] + S[c][t]
// and, with the outside score beta[c][t] = log(dS[root][0]/dS[c][t]) - ... (posterior = exp(beta + S)),
//   beta[c][t] = LSE_{a<=c}( links[a][0][c] + match[a][t-1] + beta[a][t-1],
//                            links[a][1][c] + match[a-1][t-2] + match[a][t-1] + beta[a][t-2] ).
//
// Design (latency-bound sweeps over the target positions, one workgroup of 512 threads per sentence and sweep): the
// sentence's compact link matrices live in registers for the whole sweep (one 8-lane group per node, lanes strided over
// the other index), the current column of S (or of the outside weights) is exchanged through LDS, one workgroup barrier
// per target position.  The forward leaves F0/F1 behind so that the backward needs a single outside sweep; that sweep
// reads links, emissions and its own earlier columns only, so in the single call the two run side by side as two
// workgroups (inside_pair_ml1_kernel) and a parallel kernel multiplies their tables into the posteriors
// (inside_combine_ml1_kernel); in the two-call API the outside sweep accumulates rule posteriors in registers and
// emission posteriors come from an element-wise epilogue.
// Graphs of more than 130 nodes use the streaming or the pipelined sweeps (link rows from L2, or spread over several
// workgroups per sentence).
#include "common.hip.h"
#include "glat_glue.hip.h"

#include <atomic>
#include <mutex>

namespace pcfgnat {
namespace {

constexpr int NT = 1024;       // threads per sentence

__device__ __forceinline__ float sanitize(float v) { return (v != v) ? NEG_INF_F : v; }

// Column offsets.  Entries of S grow like (tokens left) x (log-probability per token), thousands for long sentences,
// where fp32 resolves only ~1e-4 - and posteriors are exponentials of sums of such entries.  Every sweep therefore
// keeps column t of the inside table relative to a per-column offset O_t (S[a][t] = R_t[a] + O_t), chosen on the fly as
// O_{t-1} = O_t + D_t with D_t following the column maximum (max_a R_t[a] in the streaming kernels, max_a R_{t+1}[a] in
// the register-resident ones, whose reduction thus stays off the critical path; any D_t is exact, the choice only bounds
// magnitudes), so that all stored and exchanged numbers stay within a few tens of units and only the offsets
// (accumulated in double) are large.  The tables the backward consumes are kept in this
// relative form:  F0h_t[a] = LSE_c(links[a][0][c] + R_t[c]) - D_t  (= F0[a][t] - O_{t-1}),  same for F1h, and the
// outside sweep produces Bh_t[c] = beta[c][t] + O_t, so that log-posteriors are sums of small numbers:
//   emission  (a,s), null left child:  Bh_s[a] + match[a][s] + F0h_{s+1}[a]
//   emission  (a,s), leaf emitted s:   Bh_s[a] + match[a-1][s] + match[a][s+1] + F1h_{s+2}[a] - D_{s+1}
//   rule      a -> c at column t:      links[a][k][c] + Wk_t[a] + R_t[c],   W0_t[a] = match[a][t-1] + Bh_{t-1}[a] - D_t,
//                                      W1_t[a] = match[a-1][t-2] + match[a][t-1] + Bh_{t-2}[a] - D_t - D_{t-1}.
//
// Aux layout per sentence (Mc <= 64): the column offsets of the forward sweep O [T+4] and of an outside sweep that ran beside
// it P [T+4] (doubles), then F0h, F1h, Bh, R, each [Mc][T+2], the forward's shifts D [T+4], the outside weights W0h, W1h
// [Mc][T+2] and the outside sweep's shifts E [T+4]; log-domain values in base 2.  The buffer must be 8-byte aligned.
__host__ __device__ inline size_t aux_stride_reg(int Mc, int T) { return (size_t)6 * Mc * (T + 2) + (size_t)6 * (T + 4); }
struct AuxView {
    double *O, *P;
    float *F0, *F1, *BETA, *SR, *D, *W0, *W1, *E;
    __device__ AuxView(float *aux, int b, int Mc, int T) {
        size_t plane = (size_t)Mc * (T + 2);
        float *base = aux + (size_t)b * aux_stride_reg(Mc, T);
        O = reinterpret_cast<double *>(base);
        P = O + (T + 4);
        base += 4 * (T + 4);
        F0 = base;
        F1 = base + plane;
        BETA = base + 2 * plane;
        SR = base + 3 * plane;
        D = base + 4 * plane;
        W0 = D + (T + 4);
        W1 = W0 + plane;
        E = W1 + plane;
    }
};

// Head of the dynamic LDS of the register-resident kernels: per-wave column maxima slots[2][8] (16-byte aligned), the
// column offsets O [T+2] (double) and the shifts D [T+4].
__host__ __device__ inline int head_floats(int T) { return 16 + 2 * (T + 2) + (T + 4); }
struct LdsHead {
    float *slots, *D;
    double *O;
    float *rest;
    __device__ LdsHead(float *smem, int T) {
        slots = smem;
        O = reinterpret_cast<double *>(smem + 16);
        D = smem + 16 + 2 * (T + 2);
        rest = smem + head_floats(T);
    }
};

__device__ __forceinline__ bool lengths_ok(int m, int n, int L, int T) {
    return m >= 4 && m <= L && (m % 2) == 0 && n >= 2 && n <= T;
}

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
// Forward and outside sweep side by side (graphs of up to 130 nodes).  The outside recurrence (see the top of this file)
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
                                                                float *__restrict__ lgrad, int L, int T, int Mc, Seed seed) {
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

// ------------------------------------------------------------------------------------------------------------
// Best tree (pcfg_best_tree.cu:64-197, 239-301): a single top-down chain per sentence, walked by one wave64.
// Candidate order for exact ties: lane = (c_id - a_id - 1) & 3 with priority 0 > 2 > 1 > 3, then c ascending, then
// (j=0,k=0) before (j=1,k=1).
// ------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ int tie_key(int rel_c, int j) {
    const int lane = rel_c & 3;
    const int rank = ((lane & 1) << 1) | (lane >> 1);  // 0, 2, 1, 3 -> 0, 1, 2, 3
    return (rank << 24) | (rel_c << 1) | j;
}

// 1024 threads stage the sentence's inside table and its emissions (MODE >= 1) and its compact link matrices (MODE 2) in
// LDS; the first wave then walks the chain without touching global memory.  MODE 0 reads everything from global memory
// (tables too large for LDS).  Dynamic LDS: S [Mc][T+2], main/leaf emissions [Mc][T] each, matrices [2][Mc][Mc].
constexpr int BT_NT = 1024;
template <int MODE>
__device__ __forceinline__ void best_tree_ml1_block(const int b, const float *__restrict__ S, const float *__restrict__ match_all,
                                                    const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                    const int64_t *__restrict__ tgt_len, int64_t *__restrict__ tree, int L, int T,
                                                    int Mc, float *smem, int *tree_lds = nullptr) {
    // tree_lds: the alignment goes to this array in LDS (which the caller has filled with -1) instead of to `tree`
    constexpr bool TAB_LDS = MODE >= 1, LINKS_LDS = MODE == 2;
    const int TS = T + 2;
    float *sS = smem;                  // [Mc][TS]
    float *sMain = sS + Mc * TS;       // [Mc][T]
    float *sLeaf = sMain + Mc * T;     // [Mc][T]
    float *sA0 = sLeaf + Mc * T;       // [Mc][Mc]  (LINKS_LDS)
    float *sA1 = sA0 + (LINKS_LDS ? Mc * Mc : 0);
    const int tid = threadIdx.x, lane = tid & 63;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *lk = links + (size_t)b * L * 2 * L;
    const float *Sb = S + (size_t)b * Mc * TS;
    int64_t *tr = tree + (size_t)b * L;
    if (tree_lds == nullptr)
        for (int i = tid; i < L; i += BT_NT) tr[i] = -1;
    const bool valid = lengths_ok(m, n, L, T);  // (a sentence that fails keeps its tree of -1: the loops below are empty for it)
    const int mc = valid ? m / 2 : 0;
    if (TAB_LDS) {  // (loops unrolled so that several loads are in flight per thread)
#pragma unroll 4
        for (int i = tid; i < mc * TS; i += BT_NT) sS[i] = Sb[i];
#pragma unroll 4
        for (int i = tid; i < mc * T; i += BT_NT) {
            const int a_id = i / T, t = i - a_id * T;
            sMain[i] = mt[(size_t)(2 * a_id + 1) * T + t];
            sLeaf[i] = mt[(size_t)(2 * a_id) * T + t];
        }
    }
    auto s_at = [&](int c_id, int t) -> float { return TAB_LDS ? sS[c_id * TS + t] : Sb[(size_t)c_id * TS + t]; };
    auto main_at = [&](int x_id, int t) -> float { return TAB_LDS ? sMain[x_id * T + t] : mt[(size_t)(2 * x_id + 1) * T + t]; };
    auto leaf_at = [&](int x_id, int t) -> float { return TAB_LDS ? sLeaf[x_id * T + t] : mt[(size_t)(2 * x_id) * T + t]; };
    if (LINKS_LDS) {
#pragma unroll 4
        for (int i = tid; i < mc * mc; i += BT_NT) {
            const int a_id = i / mc, c_id = i - a_id * mc;
            const size_t row = (size_t)(2 * a_id + 1) * 2;
            sA0[a_id * Mc + c_id] = lk[(row + 0) * L + 2 * c_id + 1];
            sA1[a_id * Mc + c_id] = lk[(row + 1) * L + 2 * c_id + 1];
        }
    }
    __syncthreads();  // orders the -1 fill of `tree` before the chain's stores as well
    if (tid >= 64 || !valid) return;
    int a_id = 0, s = 0;
    // Every marked cell (a, s) has s <= n by construction; the loop is bounded by the number of main-chain nodes.  A hop is
    // one chain of dependent steps for a single wave (operands, two candidates per lane, wave arg max, the next cell), so
    // it is written without branches: every operand is read whatever the cell's case, from an address that exists, and
    // the case only picks what counts.
    for (int hop = 0; hop < mc; hop++) {
        const int a = 2 * a_id + 1;
        const bool j0 = s < n, j1 = (n - s > 1) && a_id >= 1;
        const int t0 = min(s, T - 1), t1 = min(s + 1, T - 1), u1 = min(s + 1, TS - 1), u2 = min(s + 2, TS - 1);
        const float ma_s = main_at(a_id, t0), ml_s = leaf_at(a_id, t0), ma_s1 = main_at(a_id, t1);  // (counted only under j0 / j1)
        float best = NEG_INF_F;
        int best_key = 0x7fffffff;
        for (int c0 = a_id + 1; c0 < mc; c0 += 64) {  // one round for graphs of up to 130 nodes
            const int c_id = c0 + lane;
            const bool in = c_id < mc;
            const int cc = in ? c_id : a_id, c = 2 * cc + 1;
            const float l0 = LINKS_LDS ? sA0[a_id * Mc + cc] : lk[((size_t)a * 2 + 0) * L + c];
            const float l1 = LINKS_LDS ? sA1[a_id * Mc + cc] : lk[((size_t)a * 2 + 1) * L + c];
            const float s1 = s_at(cc, u1), s2 = s_at(cc, u2);
            // j = 0, null left child: ((links + S) + C[0][s][0]) + match, C = 0
            float v0 = ((l0 + s1) + 0.f) + ma_s;
            // j = 1, leaf a-1 emits s: ((links + S) + match[a-1][s]) + match[a][s+1]
            float v1 = ((l1 + s2) + ml_s) + ma_s1;
            v0 = (in && j0 && v0 == v0) ? v0 : NEG_INF_F;  // (a NaN never wins)
            v1 = (in && j1 && v1 == v1) ? v1 : NEG_INF_F;
            const int key0 = tie_key(c_id - a_id - 1, 0);
            const bool take1 = v1 > v0;  // equal values: j = 0 comes first
            const float v = take1 ? v1 : v0;
            const int key = take1 ? (key0 | 1) : key0;
            const bool better = (v > best) | ((v == best) & (v != NEG_INF_F) & (key < best_key));
            best = better ? v : best;
            best_key = better ? key : best_key;
        }
        // wave arg max: the maximum first, then the smallest tie key among the lanes that hold it
        const float top = wave_max(best);
        const int key = wave_min((best == top && best != NEG_INF_F) ? best_key : 0x7fffffff);
        const bool found = key != 0x7fffffff;
        const int best_j = found ? (key & 1) : 0;
        const int best_c = found ? a_id + 1 + ((key >> 1) & 0x7fffff) : -1;
        // lane 0 marks the node (pcfg_best_tree.cu:182), lane 1 its leaf where that emits: cell (b, s, 1), :268-297 with i < n-gap-1
        const bool leaf = best_c >= 0 && best_j == 1 && s < n - 2;
        if (lane == 0 || (lane == 1 && leaf)) {
            const int node = a - lane, at = lane == 0 ? s + best_j : s;
            if (tree_lds != nullptr) tree_lds[node] = at;  // for the work that follows in the same workgroup, which fills it with -1 first
            else tr[node] = at;
        }
        if (best_c < 0) break;
        a_id = best_c;
        s = s + best_j + 1;
    }
}

template <int MODE>
__global__ __launch_bounds__(BT_NT) void best_tree_ml1_kernel(const float *__restrict__ S, const float *__restrict__ match_all,
                                                             const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                             const int64_t *__restrict__ tgt_len, int64_t *__restrict__ tree, int L,
                                                             int T, int Mc) {
    extern __shared__ float smem[];
    best_tree_ml1_block<MODE>((int)blockIdx.x, S, match_all, links, out_len, tgt_len, tree, L, T, Mc, smem);
}

// The GLAT pass's form: the workgroup that has walked the sentence's tree goes on with everything the criterion does
// with the alignment (glat_glue_block).  What that work reads besides the alignment is requested before the walk (per
// node into registers, the targets into LDS), and the walk leaves the alignment in LDS (the glue writes it out, clipped),
// so that nothing waits for global memory once the walk has ended.  Dynamic LDS: the tables (table_floats, even), then the glue's 2 L
// floats, the alignment [L] and, 8-byte aligned, the targets [T] as int64.
template <int MODE>
__global__ __launch_bounds__(BT_NT) void best_tree_glue_ml1_kernel(const float *__restrict__ S, const float *__restrict__ match_all,
                                                                  const float *__restrict__ links, const int64_t *__restrict__ out_len,
                                                                  const int64_t *__restrict__ tgt_len, int L, int T, int Mc,
                                                                  int table_floats, GlatGlueArgs glue) {
    extern __shared__ float smem[];
    const int b = blockIdx.x, tid = threadIdx.x;
    float *glue_dyn = smem + table_floats;
    int *s_raw = reinterpret_cast<int *>(glue_dyn + 2 * L);
    int64_t *s_tg = reinterpret_cast<int64_t *>(s_raw + L + (L & 1));
    const GlatGlueEarly early = glat_glue_early(b, glue);
    // the targets travel in registers of the waves that do not walk and reach LDS while the first wave walks (stored ahead
    // of the tables, their arrival would be one more trip to memory in front of the walk)
    constexpr int CARRIERS = BT_NT - 64;
    const int ti = tid - 64;
    const int64_t tg0 = glue.targets[(size_t)b * T + ((ti >= 0 && ti < T) ? ti : 0)];
    for (int i = tid; i < L; i += BT_NT) s_raw[i] = -1;
    best_tree_ml1_block<MODE>(b, S, match_all, links, out_len, tgt_len, nullptr, L, T, Mc, smem, s_raw);  // (has a barrier ahead of the walk)
    if (ti >= 0) {
        if (ti < T) s_tg[ti] = tg0;
        for (int i = ti + CARRIERS; i < T; i += CARRIERS) s_tg[i] = glue.targets[(size_t)b * T + i];
    }
    __syncthreads();
    glat_glue_block<BT_NT>(b, glue, glue_dyn, &early, s_raw, s_tg);
}

// ------------------------------------------------------------------------------------------------------------
// Streaming variants for longer graphs (Mc > 64; the redo path of the pipelined sweeps up to 512 nodes and the only path
// beyond): same sweeps, but the link
// values are fetched from L2 every step (forward: straight from `links`; backward: from a compact transposed copy
// so that lanes read consecutive parents), rows are processed in tiles of 64, and the row reductions are online
// log-sum-exps over chunks of children.  Rule posteriors are produced by a separate, fully parallel kernel from the
// outside weights the sweep leaves behind.
// All tables are relative to the column offsets described at the top of this file (natural logarithms here).
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

// ------------------------------------------------------------------------------------------------------------
// Pipelined sweeps (64 < Mc <= 512): a sentence's nodes are cut into blocks of 16, one
// workgroup per block: four compute waves (16 lanes per node, the node's two link rows in registers for the whole sweep,
// NQ = MP/64 float4 per lane and plane) and one collector wave.  One workgroup per sentence is bound by the instruction
// issue of one compute unit and by fetching the link rows from L2 for every column; here every block has a compute
// unit of its own.
//
// The link matrices are triangular - a node combines children c >= a only - so block k of the forward sweep needs
// the column entries of the blocks above it and nothing from below: the top block runs free, and every other block
// follows the one above at the distance of one exchange through memory.  That latency (about a microsecond) is paid
// once per block as a skew of the pipeline, not once per column as it would be if all blocks advanced in lock step.
// The outside sweep (parents a <= c) runs the same way with the lowest block leading.
//
// Exchange: one table entry per (column, node), written once per launch with a device-scope store by the owner and read
// with device-scope loads by the collector waves of the blocks that follow; compact_links_ml1_kernel fills the tables
// with an impossible bit pattern (all ones) first, which marks an entry that has not arrived.  The collector works one
// column ahead of the compute waves (the two meet at the one LDS barrier per column), so an entry that is already
// there costs the compute waves nothing.
//
// Column offsets: a block sees only its own and the leading blocks' part of a column, so every block chooses its own
// shifts (maximum of what it saw of the previous column) and keeps its own offsets; what it publishes in the forward
// sweep are absolute values (offset added, as doubles), which the readers bring to their own offsets.  The tables a
// block leaves behind (R, F0h, F1h) are relative to its own offsets; pipeline_rebase_kernel then moves them to the
// offsets of block 0, which saw every column whole and whose shifts are the ones stored in D.  The outside sweep works
// on those common offsets throughout.
//
// The wait for an entry is bounded: after spin_limit rounds of polling (or when another block of the sentence has
// given up) the block raises the sentence's flag and leaves; the one-workgroup streaming sweep, launched right behind
// with only_flagged set, then redoes that sentence from scratch.  Leading blocks have the lower workgroup indices, so
// that with in-order dispatch a block never waits for one that has not been started.
// ------------------------------------------------------------------------------------------------------------
constexpr int NLP = 16;             // nodes per block
constexpr int NTP = 16 * NLP + 64;  // four compute waves and the collector wave
// stream_row_lse on link rows held in registers: chunks q in [qa, qb) of the NQ the lane holds (both wave-uniform).
template <int NQ, bool JOINT>
__device__ __forceinline__ void slab_row_lse(const float4 (&A0)[NQ], const float4 (&A1)[NQ], const float4 *u0, const float4 *u1, int qa,
                                             int qb, bool live, bool has1, float g, float &out0, float &out1) {
    g = is_finite(g) ? g : 0.f;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        if (q >= qa && q < qb) {
            const float4 c0 = minus(u0[16 * q], g);
            const float4 c1 = JOINT ? minus(u1[16 * q], g) : c0;
            s0 += sum4_ex2(A0[q], c0);
            s1 += sum4_ex2(A1[q], c1);
        }
    }
    bool ok;
    if (JOINT) {
        const float tot = node_sum<16>(s0 + s1);
        ok = tot >= 0x1p-90f && tot <= 0x1p100f;
        out0 = g + lg2(tot);
        out1 = out0;
    } else {
        const float t0 = node_sum<16>(s0), t1 = node_sum<16>(s1);
        ok = t0 >= 0x1p-90f && t0 <= 0x1p100f && ((t1 >= 0x1p-90f && t1 <= 0x1p100f) || !has1);
        out0 = g + lg2(t0);
        out1 = has1 ? g + lg2(t1) : NEG_INF_F;
    }
    if (live && !ok) {  // uniform over the lanes of the node
        RunningLse<16> a0, a1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q >= qa && q < qb) {
                const float4 c0 = u0[16 * q];
                const float4 c1 = JOINT ? u1[16 * q] : c0;
                a0.add4(A0[q], c0);
                a1.add4(A1[q], c1);
            }
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

template <bool MATCH_LDS, int SL>
__global__ __launch_bounds__(NT) void inside_bwd_ml1_stream_kernel(const float *__restrict__ S, float *__restrict__ aux,
                                                                  const float *__restrict__ match_all,
                                                                  const int64_t *__restrict__ out_len,
                                                                  const int64_t *__restrict__ tgt_len, int L, int T, int Mc, int MP,
                                                                  int only_flagged) {
    if (only_flagged) {
        if (ExchangeView(aux, blockIdx.x, Mc, T).flags[FLAG_BWD] == 0) return;
        if (threadIdx.x == 0) atomicAdd(&g_inside_redone, 1ull);
    }
    extern __shared__ float smem[];
    inside_bwd_ml1_stream_block<MATCH_LDS, SL>((int)blockIdx.x, S, aux, match_all, out_len, tgt_len, L, T, Mc, MP, smem);
}

// Both sweeps' second chance in one launch, after the pipelines that ran side by side: grid (B, 2), workgroup (b, 0)
// sweeps sentence b forward again if its forward pipeline gave up, workgroup (b, 1) its outside sweep if that pipeline
// gave up.  The outside sweep reads the forward's column shifts and log-likelihood: where both are redone, its workgroup
// waits for the forward's, which was dispatched before it (x runs fastest) and waits for nobody; the forward's tables
// reach it through a device-scope release / acquire pair around the flag FLAG_FWD_REDONE (the two workgroups may sit on
// different L2s).  In the normal case neither flag is set and the launch ends at once - one launch where two stood.
// Dynamic LDS: the larger of the two sweeps' needs without the emissions.
constexpr int FLAG_FWD_REDONE = 2;
// set where the second chance of a sentence was given up: pipeline_finish_kernel, the next launch, then turns the
// sentence's log-likelihood into NaN (not this launch: the forward's workgroup may still be writing it)
constexpr int FLAG_GIVEN_UP = 3;
template <int SLB>
__global__ __launch_bounds__(NT) void inside_redo_ml1_stream_kernel(const float *match_all, const float *links, const int64_t *out_len,
                                                                   const int64_t *tgt_len, float *S, float *aux, int L, int T, int Mc,
                                                                   int MP, int wait_limit) {
    extern __shared__ float smem[];
    const int b = blockIdx.x;
    int *flags = ExchangeView(aux, b, Mc, T).flags;
    if (blockIdx.y == 0) {
        if (flags[FLAG_FWD] == 0) return;
        if (threadIdx.x == 0) atomicAdd(&g_inside_redone, 1ull);
        inside_fwd_ml1_stream_block<false, 4>(b, match_all, links, out_len, tgt_len, S, aux, L, T, Mc, MP, smem);
        __threadfence();  // every thread's table entries are out before the flag
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_store(flags + FLAG_FWD_REDONE, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    if (flags[FLAG_BWD] == 0) return;
    if (threadIdx.x == 0) atomicAdd(&g_inside_redone, 1ull);
    if (flags[FLAG_FWD] != 0) {
        __shared__ int s_arrived;
        if (threadIdx.x == 0) {
            // The forward's workgroup is running or done and waits for nobody, so this wait ends; it is bounded all the
            // same (seconds), like every wait between workgroups here.  Past the bound the sentence is given up: the next
            // launch turns its log-likelihood into NaN, which the posterior kernels and the loss treat as an invalid sentence.
            int arrived = 0;
            for (int spins = 0; spins < wait_limit && !arrived; spins++) {
                arrived = __hip_atomic_load(flags + FLAG_FWD_REDONE, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) != 0;
                if (!arrived) __builtin_amdgcn_s_sleep(16);
            }
            s_arrived = arrived;
            if (!arrived) {
                flags[FLAG_GIVEN_UP] = 1;
                atomicAdd(&g_inside_given_up, 1ull);
            }
        }
        __syncthreads();
        if (!s_arrived) return;
        __threadfence();
    }
    inside_bwd_ml1_stream_block<false, SLB>(b, S, aux, match_all, out_len, tgt_len, L, T, Mc, MP, smem);
}

// Forward sweep of one block.  Same tables as inside_fwd_ml1_stream_kernel, relative to the block's own offsets (see
// above).  Dynamic LDS (MATCH_LDS): the emissions of the block's nodes, main [NLP][T] and leaf [NLP][T]; without it they
// are requested one column ahead.
template <int NQ, bool MATCH_LDS, int CW>
__device__ __forceinline__ void inside_fwd_ml1_pipe_body(const int bid, const float *__restrict__ match_all,
                                                        const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                        float *__restrict__ S, float *__restrict__ aux, int L, int T, int Mc,
                                                        int spin_limit) {
    constexpr int MP = 64 * NQ, CL = MP / NLP;
    __shared__ __attribute__((aligned(16))) float col[2][MP];
    __shared__ float sm_Dv[2][4];  // shift of the step that reads column t: maximum of the visible part of column t+1, one
                                   // partial maximum per collector wave
    __shared__ int sm_dead;
    extern __shared__ float sm_match[];
    float *sm_main = sm_match, *sm_leaf = sm_match + NLP * T;
    const int b = bid / CL, k = CL - 1 - bid % CL;  // the leading (highest) block first
    const int tid = threadIdx.x, gidx = (tid >> 4) & (NLP - 1), j = tid & 15, lane = tid & 63;
    // CW collector waves behind the compute waves (see outside_free_ml1_pipe_body): wave cw takes the chunks cw, cw+CW, ..
    const bool collector = tid >= 16 * NLP, compute = !collector;
    const int cw = (CW == 1) ? 0 : ((tid >> 6) & 3);
    constexpr int NR = (NQ + CW - 1) / CW;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    float *Sb = S + (size_t)b * Mc * (T + 2);
    AuxViewStream av(aux, b, Mc, T);
    ExchangeView xv(aux, b, Mc, T);
    const int part = (bid % CL) * NTP + tid, nparts = CL * NTP;  // the sentence's element-wise work is split over the blocks

    if (!lengths_ok(m, n, L, T)) {
        for (int i = part; i < Mc * (T + 2); i += nparts) Sb[i] = (i == 0) ? __builtin_nanf("") : NEG_INF_F;
        return;
    }
    const int mc = m / 2;
    for (int i = part; i < Mc * (T + 2); i += nparts) {
        const int a_id = i / (T + 2), s = i - a_id * (T + 2);
        if (a_id >= mc || s >= n - 1) {
            float v = NEG_INF_F;
            if (a_id == mc - 1 && s == n - 1) v = sanitize(mt[(size_t)(m - 1) * T + (n - 1)]);
            Sb[i] = v;
            av.SR[i] = v * LOG2E_F;
        }
    }
    if (k == 0)
        for (int i = tid; i < T + 4; i += NTP) av.D[i] = 0.f;
    if (NLP * k >= mc) return;  // no node of the sentence in this block: nobody waits for it
    const float base_cell = to_b2(mt[(size_t)(m - 1) * T + (n - 1)]);
    for (int i = tid; i < 2 * MP; i += NTP) (&col[0][0])[i] = NEG_INF_F;
    __syncthreads();
    if (tid == 0) {
        col[(n - 1) & 1][mc - 1] = base_cell;
        sm_dead = 0;
    }
    if (tid < 8) (&sm_Dv[0][0])[tid] = (tid & 3) ? NEG_INF_F : 0.f;  // slots of absent collector waves stay at -inf

    // this lane's node and its link rows (rows beyond the sentence: any valid row, the result is discarded)
    const int a_id = NLP * k + gidx;
    const bool row_ok = a_id < mc;
    const int ar = row_ok ? a_id : NLP * k;
    const int q0 = (NLP * k) / 64;  // the chunk that holds the block's diagonal
    float4 A0[NQ], A1[NQ];
    if (compute) {
        const float4 *r0 = reinterpret_cast<const float4 *>(av.Ac + ((size_t)0 * Mc + ar) * MP) + j;
        const float4 *r1 = reinterpret_cast<const float4 *>(av.Ac + ((size_t)1 * Mc + ar) * MP) + j;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            A0[q] = r0[16 * q];
            A1[q] = r1[16 * q];
        }
    }
    const float *ra = mt + (size_t)(2 * ar + 1) * T, *rl = mt + (size_t)(2 * ar) * T;
    if (MATCH_LDS) {
        for (int i = tid; i < NLP * T; i += NTP) {
            const int g = i / T, s = i - g * T, node = NLP * k + g;
            const bool ok = node < mc && s < n;
            sm_main[i] = ok ? to_b2(mt[(size_t)(2 * node + 1) * T + s]) : NEG_INF_F;
            sm_leaf[i] = (ok && node >= 1) ? to_b2(mt[(size_t)(2 * node) * T + s]) : NEG_INF_F;
        }
        __syncthreads();
    }
    float ma_t = MATCH_LDS ? sm_main[gidx * T + n - 1] : to_b2(ra[n - 1]);                        // main[a][t]
    float ma_p = MATCH_LDS ? sm_main[gidx * T + n - 2] : to_b2(ra[n - 2]);                        // main[a][t-1]
    float ml_p = MATCH_LDS ? sm_leaf[gidx * T + n - 2] : (ar >= 1 ? to_b2(rl[n - 2]) : NEG_INF_F);  // leaf[a][t-1]
    float f0g = NEG_INF_F, f1p = NEG_INF_F;                  // the node's F0, F1 one column earlier
    // The link rows must have arrived before the sweep starts: a wait for them inside the loop would, from the second
    // column on, be a wait for the stores of the column before.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    unsigned long long *Xf = xv.fcol;
    float *Dk = xv.shifts + (size_t)k * (T + 4);
    const unsigned long long MINUS_INF64 = (unsigned long long)__double_as_longlong(-__builtin_huge_val());
    unsigned long long x[NR];  // collectors: the entries of the blocks above, requested one step before they are handed on
#pragma unroll
    for (int ri = 0; ri < NR; ri++) {
        const int r = cw + CW * ri, i = NLP * (k + 1) + 64 * min(r, NQ - 1) + lane;
        x[ri] = (collector && n >= 3 && r < NQ) ? entry_load(Xf + (size_t)(n - 2) * MP + i) : MINUS_INF64;
    }
    double O = 0.0;  // offset of the column being read
    for (int t = n - 1; t >= 1; t--) {
        const float *cur = col[t & 1];
        float *nxt = col[(t - 1) & 1];
        const float D = fmaxf(fmaxf(sm_Dv[t & 1][0], sm_Dv[t & 1][1]), fmaxf(sm_Dv[t & 1][2], sm_Dv[t & 1][3]));
        const float Ds = (D == NEG_INF_F) ? 0.f : D;
        const double O_new = O + (double)Ds;  // offset of column t-1
        if (collector) {
            if (t > 1) {  // column t-1 of the blocks above, requested one iteration ago
                const unsigned long long *src = Xf + (size_t)(t - 1) * MP + NLP * (k + 1) + lane;
                // the requests went out for every lane (a branch around a load ends in a wait for it); entries beyond the
                // sentence are never written and read as -inf
#pragma unroll
                for (int ri = 0; ri < NR; ri++)
                    if (cw + CW * ri >= NQ || NLP * (k + 1) + 64 * (cw + CW * ri) + lane >= mc) x[ri] = MINUS_INF64;
                for (int spins = 0;; spins++) {
                    bool pending = false;
#pragma unroll
                    for (int ri = 0; ri < NR; ri++) pending |= (x[ri] == EMPTY64);
                    if (!__any(pending)) break;
                    if (spins >= spin_limit || ((spins & 63) == 63 && gave_up(xv.flags + FLAG_FWD))) {
                        sm_dead = 1;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(2);  // leave the issue slots of this SIMD to its compute wave
#pragma unroll
                    for (int ri = 0; ri < NR; ri++)
                        if (x[ri] == EMPTY64) x[ri] = entry_load(src + 64 * min(cw + CW * ri, NQ - 1));
                }
#pragma unroll
                for (int ri = 0; ri < NR; ri++) {
                    const int r = cw + CW * ri, i = NLP * (k + 1) + 64 * r + lane;
                    if (r < NQ && i < MP) nxt[i] = (x[ri] == EMPTY64) ? NEG_INF_F : (float)(__longlong_as_double((long long)x[ri]) - O_new);
                }
            }
            if (t > 2) {  // request column t-2 now: it has the whole next step to arrive
#pragma unroll
                for (int ri = 0; ri < NR; ri++)
                    x[ri] = entry_load(Xf + (size_t)(t - 2) * MP + NLP * (k + 1) + 64 * min(cw + CW * ri, NQ - 1) + lane);
            }
            // the shift of the next step from the visible part of column t, which is complete
            float vm = NEG_INF_F;
#pragma unroll
            for (int ri = 0; ri < NR; ri++) {
                const int r = cw + CW * ri, i = NLP * k + 64 * r + lane;
                if (r < NQ && i < MP) vm = fmaxf(vm, cur[i]);
            }
            vm = wave_max(vm);
            if (lane == 0) sm_Dv[(t - 1) & 1][cw] = vm;
        } else if (compute) {
            // the next column's emissions: from LDS, or requested now so that they travel during the column's work
            float ma_raw = 0.f, ml_raw = 0.f;
            if (t > 1) {
                ma_raw = MATCH_LDS ? sm_main[gidx * T + t - 2] : ra[t - 2];
                ml_raw = MATCH_LDS ? sm_leaf[gidx * T + t - 2] : rl[t - 2];
            }
            const float4 *cv = reinterpret_cast<const float4 *>(cur) + j;
            float F0, F1;
            slab_row_lse<NQ, false>(A0, A1, cv, cv, q0, NQ, row_ok, a_id >= 1, f0g, F0, F1);
            F0 -= Ds;
            F1 -= Ds;
            float s_new = lse2_b2(ma_p + F0, (ml_p + ma_t) + (f1p - Ds));
            if (!row_ok) s_new = NEG_INF_F;
            f1p = F1;
            f0g = F0;
            if (j == 0) {
                nxt[a_id] = s_new;
                if (row_ok) {
                    const double s_abs = (double)s_new + O_new;
                    if (t > 1) entry_store(Xf + (size_t)(t - 1) * MP + a_id, s_abs);
                    Sb[(size_t)a_id * (T + 2) + (t - 1)] = (float)(s_abs * LN2_D);
                    av.SR[(size_t)a_id * (T + 2) + (t - 1)] = s_new;
                    av.F0[(size_t)a_id * (T + 2) + t] = F0;
                    av.F1[(size_t)a_id * (T + 2) + t] = F1;
                }
            }
            if (tid == 0) {
                Dk[t] = Ds;
                if (k == 0) av.D[t] = Ds;
            }
            ma_t = ma_p;
            ma_p = MATCH_LDS ? ma_raw : to_b2(ma_raw);
            ml_p = MATCH_LDS ? ml_raw : (ar >= 1 ? to_b2(ml_raw) : NEG_INF_F);
        }
        O = O_new;
        lds_barrier();
        if (sm_dead) {  // uniform: written before the barrier
            if (tid == 0) __hip_atomic_store(xv.flags + FLAG_FWD, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
}

template <int NQ, bool MATCH_LDS, int CW = 1>
__global__ __launch_bounds__(16 * NLP + 64 * CW) void inside_fwd_ml1_pipe_kernel(const float *__restrict__ match_all,
                                                                                const int64_t *__restrict__ out_len,
                                                                                const int64_t *__restrict__ tgt_len, float *__restrict__ S,
                                                                                float *__restrict__ aux, int L, int T, int Mc,
                                                                                int spin_limit) {
    inside_fwd_ml1_pipe_body<NQ, MATCH_LDS, CW>((int)blockIdx.x, match_all, out_len, tgt_len, S, aux, L, T, Mc, spin_limit);
}

// ------------------------------------------------------------------------------------------------------------
// The two pipelined sweeps side by side (single call, graphs of 130..1026 nodes).  Like the paired sweeps of short graphs:
// the outside recurrence needs links, emissions and its own earlier columns, not the inside table, so the outside pipeline
// need not follow the forward one - provided it stops borrowing the forward's column shifts.  Here every block of the
// outside sweep chooses its own shifts (e_{t+1} = maximum of the part of the weight columns W0_{t-1}, W1_{t-1} it saw) and
// keeps offsets P_t = e_1 + .. + e_t of its own (true value = relative value + P_t); what it publishes are absolute
// weights (as doubles) which the readers bring to their own offsets, exactly as the forward sweep does with its
// columns.  pipeline_finish_kernel then moves the blocks' tables (Bh, W0, W1) to the offsets of the last block
// that holds nodes of the sentence - it saw every column whole - and writes one correction per column for the
// posterior kernels,
//   corr_t  = P_t     + O_t - ll      (rule a -> c at column t; emission with the null left child; base cell)
//   corr1_t = P_{t-1} + O_t - ll      (emissions that go through the local leaf),
// with O_t the forward's offsets; for a sentence whose outside sweep was redone on the forward's offsets by the
// one-workgroup kernel they are 0 and -D_t.
// ------------------------------------------------------------------------------------------------------------
template <int NQ, bool MATCH_LDS, int CW>
__device__ __forceinline__ void outside_free_ml1_pipe_body(const int bid, const float *__restrict__ match_all,
                                                          const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                          float *__restrict__ aux, int L, int T, int Mc, int spin_limit) {
    constexpr int MP = 64 * NQ, CL = MP / NLP;
    __shared__ __attribute__((aligned(16))) float w0[2][MP];
    __shared__ __attribute__((aligned(16))) float w1[2][MP];
    __shared__ float sm_Ev[2][4];  // shift chosen at the step that reads the columns t: maximum of the visible part of the
                                   // columns t-1, one partial maximum per collector wave
    __shared__ int sm_dead;
    extern __shared__ float sm_em[];
    float *sm_main = sm_em, *sm_leaf = sm_em + NLP * T;
    const int b = bid / CL, k = bid % CL;  // the leading (lowest) block first
    const int tid = threadIdx.x, gidx = (tid >> 4) & (NLP - 1), j = tid & 15, lane = tid & 63;
    // CW collector waves behind the compute waves (four: one per SIMD, for launches in which a block has a compute unit to
    // itself; one otherwise): wave cw takes the chunks cw, cw+CW, .. of both planes
    const bool collector = tid >= 16 * NLP;
    const int cw = (CW == 1) ? 0 : ((tid >> 6) & 3);
    constexpr int NR = (NQ + CW - 1) / CW;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    AuxViewStream av(aux, b, Mc, T);
    ExchangeView xv(aux, b, Mc, T);
    if (!lengths_ok(m, n, L, T)) return;  // the posterior kernels write zeros for such sentences
    const int mc = m / 2;
    if (NLP * k >= mc) return;  // no node of the sentence in this block: nobody waits for it
    for (int i = tid; i < 2 * MP; i += NTP) {
        (&w0[0][0])[i] = NEG_INF_F;
        (&w1[0][0])[i] = NEG_INF_F;
    }
    if (tid == 0) sm_dead = 0;
    if (tid < 8) (&sm_Ev[0][0])[tid] = (tid & 3) ? NEG_INF_F : 0.f;  // slots of absent collector waves stay at -inf
    if (MATCH_LDS) {
        for (int i = tid; i < NLP * T; i += NTP) {
            const int g = i / T, s = i - g * T, node = NLP * k + g;
            const bool ok = node < mc && s < n;
            sm_main[i] = ok ? to_b2(mt[(size_t)(2 * node + 1) * T + s]) : NEG_INF_F;
            sm_leaf[i] = (ok && node >= 1) ? to_b2(mt[(size_t)(2 * node) * T + s]) : NEG_INF_F;
        }
    }

    // this lane's node and its transposed link rows: parents a <= c, chunks [0, q1)
    const int c_id = NLP * k + gidx;
    const bool live = c_id < mc;
    const int ci = live ? c_id : NLP * k;
    const int q1 = (NLP * k + NLP - 1) / 64 + 1;
    float4 A0[NQ], A1[NQ];
    if (!collector) {
        const float4 *r0 = reinterpret_cast<const float4 *>(av.At + ((size_t)0 * Mc + ci) * MP) + j;
        const float4 *r1 = reinterpret_cast<const float4 *>(av.At + ((size_t)1 * Mc + ci) * MP) + j;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            A0[q] = r0[16 * q];
            A1[q] = r1[16 * q];
        }
    }
    const float *ra = mt + (size_t)(2 * ci + 1) * T, *rl = mt + (size_t)(2 * ci) * T;
    __syncthreads();  // the cleared columns
    // beta[root][0] = 0 with P_0 = P_1 = 0: the only weight of column 1 is the root's, match[root][0]
    const float w00 = to_b2(mt[(size_t)1 * T]);
    if (tid == 0) w0[1][0] = w00;
    float bp = (c_id == 0) ? 0.f : NEG_INF_F;  // the node's relative outside score one column earlier
    if (!collector && j == 0 && live) {
        av.BETA[(size_t)c_id * (T + 2)] = bp;
        av.W0[(size_t)c_id * (T + 2) + 1] = (c_id == 0) ? w00 : NEG_INF_F;
        av.W1[(size_t)c_id * (T + 2) + 1] = NEG_INF_F;
    }
    float mc_t, ml_p;  // main[c][t], leaf[c][t-1]
    if (MATCH_LDS) {
        mc_t = sm_main[gidx * T + 1];
        ml_p = sm_leaf[gidx * T];
    } else {
        mc_t = live ? to_b2(ra[1]) : NEG_INF_F;
        ml_p = (live && ci >= 1) ? to_b2(rl[0]) : NEG_INF_F;
    }
    // The link rows must have arrived before the sweep starts: a wait for them inside the loop would, from the second
    // column on, be a wait for the stores of the column before.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    unsigned long long *Xo = xv.obw;
    float *Ek = xv.shiftsE + (size_t)k * (T + 4);
    if (tid == 0) {
        Ek[0] = 0.f;
        Ek[1] = 0.f;
    }
    const unsigned long long MINUS_INF64 = (unsigned long long)__double_as_longlong(-__builtin_huge_val());
    unsigned long long x0[NR], x1[NR];  // collectors: the entries of the blocks below, requested one step before they are handed on
#pragma unroll
    for (int ri = 0; ri < NR; ri++) {
        const int r = cw + CW * ri;
        const bool need = collector && k > 0 && n >= 3 && r < NQ;
        x0[ri] = need ? entry_load(Xo + (size_t)2 * 2 * MP + 64 * r + lane) : MINUS_INF64;
        x1[ri] = need ? entry_load(Xo + (size_t)2 * 2 * MP + MP + 64 * r + lane) : MINUS_INF64;
    }
    double P = 0.0;      // P_t, the offset of the columns being read
    float e_cur = 0.f;   // e_t
    for (int t = 1; t <= n - 1; t++) {
        const float *c0 = w0[t & 1], *c1 = w1[t & 1];
        float *n0 = w0[(t + 1) & 1], *n1 = w1[(t + 1) & 1];
        const bool more = t < n - 1;
        const float E = fmaxf(fmaxf(sm_Ev[t & 1][0], sm_Ev[t & 1][1]), fmaxf(sm_Ev[t & 1][2], sm_Ev[t & 1][3]));
        const float e_next = is_finite(E) ? E : 0.f;  // e_{t+1}
        const double P_next = P + (double)e_next;     // P_{t+1}
        if (collector) {
            if (more && k > 0) {  // the weights of the blocks below for column t+1, requested one iteration ago
                const unsigned long long *src = Xo + (size_t)(t + 1) * 2 * MP + lane;
                // the requests went out for every lane (a branch around a load ends in a wait for it); entries of other
                // blocks' nodes beyond the sentence are never written and read as -inf
#pragma unroll
                for (int ri = 0; ri < NR; ri++) {
                    if (64 * (cw + CW * ri) + lane >= min(NLP * k, mc)) {
                        x0[ri] = MINUS_INF64;
                        x1[ri] = MINUS_INF64;
                    }
                }
                for (int spins = 0;; spins++) {
                    bool pending = false;
#pragma unroll
                    for (int ri = 0; ri < NR; ri++) pending |= (x0[ri] == EMPTY64) | (x1[ri] == EMPTY64);
                    if (!__any(pending)) break;
                    if (spins >= spin_limit || ((spins & 63) == 63 && gave_up(xv.flags + FLAG_BWD))) {
                        sm_dead = 1;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(2);  // leave the issue slots of this SIMD to its compute wave
#pragma unroll
                    for (int ri = 0; ri < NR; ri++) {
                        const int r = min(cw + CW * ri, NQ - 1);
                        if (x0[ri] == EMPTY64) x0[ri] = entry_load(src + 64 * r);
                        if (x1[ri] == EMPTY64) x1[ri] = entry_load(src + MP + 64 * r);
                    }
                }
#pragma unroll
                for (int ri = 0; ri < NR; ri++) {
                    const int r = cw + CW * ri, i = 64 * r + lane;
                    if (r < NQ && i < NLP * k) {
                        n0[i] = (x0[ri] == EMPTY64) ? NEG_INF_F : (float)(__longlong_as_double((long long)x0[ri]) - P_next);
                        n1[i] = (x1[ri] == EMPTY64) ? NEG_INF_F : (float)(__longlong_as_double((long long)x1[ri]) - P_next);
                    }
                }
            }
            if (t + 2 <= n - 1 && k > 0) {  // request column t+2 now: it has the whole next step to arrive
                const unsigned long long *src = Xo + (size_t)(t + 2) * 2 * MP + lane;
#pragma unroll
                for (int ri = 0; ri < NR; ri++) {
                    const int r = min(cw + CW * ri, NQ - 1);  // (a wave without a chunk of its own re-reads the last one and drops it)
                    x0[ri] = entry_load(src + 64 * r);
                    x1[ri] = entry_load(src + MP + 64 * r);
                }
            }
            // the shift of the next step from the visible part of the columns t, which is complete
            float vm = NEG_INF_F;
#pragma unroll
            for (int ri = 0; ri < NR; ri++) {
                const int r = cw + CW * ri, i = 64 * r + lane;
                if (r < NQ && i < NLP * (k + 1)) vm = fmaxf(vm, fmaxf(c0[i], c1[i]));
            }
            vm = wave_max(vm);
            if (lane == 0) sm_Ev[(t + 1) & 1][cw] = vm;
        } else {
            float mc_raw = 0.f, ml_raw = 0.f;
            if (more) {
                mc_raw = MATCH_LDS ? sm_main[gidx * T + t + 1] : ra[t + 1];
                ml_raw = MATCH_LDS ? sm_leaf[gidx * T + t] : rl[t];
            }
            const float4 *u0 = reinterpret_cast<const float4 *>(c0) + j, *u1 = reinterpret_cast<const float4 *>(c1) + j;
            float beta, unused;
            slab_row_lse<NQ, true>(A0, A1, u0, u1, 0, q1, live, true, bp, beta, unused);
            if (!live) beta = NEG_INF_F;
            const float nw0 = (mc_t + beta) - e_next;
            const float nw1 = ((ml_p + mc_t) + bp) - (e_next + e_cur);
            if (j == 0) {
                n0[c_id] = nw0;
                n1[c_id] = nw1;
                if (live) {
                    if (more) {
                        entry_store(Xo + (size_t)(t + 1) * 2 * MP + c_id, (double)nw0 + P_next);
                        entry_store(Xo + (size_t)(t + 1) * 2 * MP + MP + c_id, (double)nw1 + P_next);
                    }
                    av.BETA[(size_t)c_id * (T + 2) + t] = beta;
                    av.W0[(size_t)c_id * (T + 2) + t + 1] = nw0;
                    av.W1[(size_t)c_id * (T + 2) + t + 1] = nw1;
                }
            }
            if (tid == 0) Ek[t + 1] = e_next;
            bp = beta;
            mc_t = MATCH_LDS ? mc_raw : (live ? to_b2(mc_raw) : NEG_INF_F);
            ml_p = MATCH_LDS ? ml_raw : ((live && ci >= 1) ? to_b2(ml_raw) : NEG_INF_F);
        }
        e_cur = e_next;
        P = P_next;
        lds_barrier();
        if (sm_dead) {  // uniform: written before the barrier
            if (tid == 0) __hip_atomic_store(xv.flags + FLAG_BWD, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
}

// Both sweeps in one launch: the first `fwd_blocks` workgroups are the forward pipeline's, the others the outside one's
// (leading blocks first within either).
template <int NQ, bool MATCH_LDS, int CW>
__global__ __launch_bounds__(16 * NLP + 64 * CW) void inside_both_ml1_pipe_kernel(const float *__restrict__ match_all,
                                                                  const int64_t *__restrict__ out_len,
                                                                  const int64_t *__restrict__ tgt_len, float *__restrict__ S,
                                                                  float *__restrict__ aux, int L, int T, int Mc, int spin_limit,
                                                                  int spin_limit_outside, int fwd_blocks) {
    if ((int)blockIdx.x < fwd_blocks)  // workgroup-uniform
        inside_fwd_ml1_pipe_body<NQ, MATCH_LDS, CW>((int)blockIdx.x, match_all, out_len, tgt_len, S, aux, L, T, Mc, spin_limit);
    else
        outside_free_ml1_pipe_body<NQ, MATCH_LDS, CW>((int)blockIdx.x - fwd_blocks, match_all, out_len, tgt_len, aux, L, T, Mc,
                                                  spin_limit_outside);
}

// After the sweeps side by side (and the forward's redo, if any): grid (CL, B), 256 threads.  Block k < K (K = the last
// block with nodes of the sentence) moves its outside tables to block K's offsets, delta_t = P^k_t - P^K_t:
// Bh[c][t], W0[c][t], W1[c][t] += delta_t.  Block K writes the corrections corr_t, corr1_t (see above).  A sentence
// whose outside sweep gave up is redone afterwards on the forward's offsets: corr = 0, corr1_t = -D_t.
// Dynamic LDS: two rows of T+4 doubles.
// Inclusive prefix sums of v[0..len) in place (LDS, doubles) by the 256 threads of a workgroup: every thread sums a run of
// consecutive entries, the runs are chained by shuffles inside the waves and through `part` (LDS, four doubles) across
// them.  All threads must call it; barriers inside.
__device__ __forceinline__ void block_prefix_sum(double *v, int len, double *part, int tid) {
    const int run = (len + 255) / 256, lo = tid * run;
    double acc = 0.0;
    for (int i = 0; i < run; i++)
        if (lo + i < len) acc += v[lo + i];
    double incl = acc;
    for (int o = 1; o < 64; o <<= 1) {
        const double y = __shfl_up(incl, o);
        if ((tid & 63) >= o) incl += y;
    }
    if ((tid & 63) == 63) part[tid >> 6] = incl;
    __syncthreads();
    double run_sum = incl - acc;  // the entries before this thread's run
    for (int w = 0; w < (tid >> 6); w++) run_sum += part[w];
    for (int i = 0; i < run; i++) {
        if (lo + i < len) {
            run_sum += v[lo + i];
            v[lo + i] = run_sum;
        }
    }
    __syncthreads();
}

__device__ __forceinline__ void pipeline_finish_outside_block(const int k, const int b, float *__restrict__ aux,
                                                              const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                              int L, int T, int Mc, double *sm_row) {
    __shared__ double sm_part[4];
    double *sm_a = sm_row, *sm_b = sm_row + (T + 4);
    const int tid = threadIdx.x;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    if (!lengths_ok(m, n, L, T)) return;
    const int mc = m / 2, K = (mc - 1) / NLP, CLEN = corr_len(T);
    if (k > K) return;
    AuxViewStream av(aux, b, Mc, T);
    ExchangeView xv(aux, b, Mc, T);
    const bool redo = xv.flags[FLAG_BWD] != 0;
    const float *EK = xv.shiftsE + (size_t)K * (T + 4);
    if (k == K) {
        if (redo) {
            for (int t = tid; t < CLEN; t += 256) {
                xv.corr[t] = 0.f;
                xv.corr[CLEN + t] = (t < T + 4) ? -av.D[t] : 0.f;
            }
            return;
        }
        // sm_a[t] = P_t = e_1 + .. + e_t; sm_b[u] = D_{n-1} + .. + D_{n-1-u}, so that O_t = sm_b[n-2-t] (O_{n-1} = 0)
        for (int t = tid; t < n; t += 256) {
            sm_a[t] = (t >= 1) ? (double)EK[t] : 0.0;
            sm_b[t] = (n - 1 - t >= 1) ? (double)av.D[n - 1 - t] : 0.0;
        }
        __syncthreads();
        block_prefix_sum(sm_a, n, sm_part, tid);
        block_prefix_sum(sm_b, n, sm_part, tid);
        const double O0 = (n >= 2) ? sm_b[n - 2] : 0.0;
        const double ll_abs = (double)av.SR[0] + O0;
        for (int t = tid; t < CLEN; t += 256) {
            const bool in = t <= n - 1;
            const double Ot = (in && t <= n - 2) ? sm_b[n - 2 - t] : 0.0;
            xv.corr[t] = in ? (float)(sm_a[t] + Ot - ll_abs) : 0.f;
            xv.corr[CLEN + t] = (in && t >= 1) ? (float)(sm_a[t - 1] + Ot - ll_abs) : 0.f;
        }
        return;
    }
    if (redo) return;
    const float *Ek = xv.shiftsE + (size_t)k * (T + 4);
    for (int t = tid; t < n; t += 256) sm_a[t] = (t >= 1) ? (double)Ek[t] - (double)EK[t] : 0.0;
    __syncthreads();
    block_prefix_sum(sm_a, n, sm_part, tid);  // delta_t
    const int TS = T + 2, cells = NLP * TS;
    for (int base = tid; base < cells; base += 4 * 256) {  // four cells per thread in flight
        float bv[4], v0[4], v1[4];
        size_t o[4];
        int tc[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = base + u * 256, g = i / TS, t = i - g * TS, c_id = NLP * k + g;
            const bool ok = i < cells && c_id < mc && t <= n - 1;
            tc[u] = ok ? t : -1;
            o[u] = (size_t)(ok ? c_id : NLP * k) * TS + (ok ? t : 0);
            bv[u] = av.BETA[o[u]];
            v0[u] = av.W0[o[u]];
            v1[u] = av.W1[o[u]];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int t = tc[u];
            if (t >= 0) av.BETA[o[u]] = (float)((double)bv[u] + sm_a[t]);
            if (t >= 1) {
                av.W0[o[u]] = (float)((double)v0[u] + sm_a[t]);
                av.W1[o[u]] = (float)((double)v1[u] + sm_a[t]);
            }
        }
    }
}

// Moves the tables of blocks 1 .. CL-1 from their own column offsets to those of block 0 (see above): with
// O_s = sum_{t > s} D_t, R[a][s] is relative to O_s and F0h[a][t], F1h[a][t] to O_{t-1}.  Grid (CL-1, B).
__device__ __forceinline__ void pipeline_rebase_block(const int k, const int b, float *__restrict__ aux,
                                                      const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len, int L,
                                                      int T, int Mc, double *sm_delta) {
    __shared__ double sm_part[4];
    const int tid = threadIdx.x;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    if (!lengths_ok(m, n, L, T)) return;
    const int mc = m / 2;
    if (NLP * k >= mc) return;
    AuxViewStream av(aux, b, Mc, T);
    ExchangeView xv(aux, b, Mc, T);
    if (xv.flags[FLAG_FWD] != 0) return;  // the sentence is redone from scratch
    const float *Dk = xv.shifts + (size_t)k * (T + 4), *D0 = xv.shifts;
    // delta[s] = sum_{t = s+1}^{n-1} (Dk[t] - D0[t]): every thread sums a run of columns, the runs are then chained
    const int run = (n + 255) / 256;  // columns per thread
    const int hi = n - 1 - tid * run;  // this thread's columns: hi, hi-1, ..., hi-run+1 (those >= 1)
    double acc = 0.0;
    for (int i = 0; i < run; i++) {
        const int t = hi - i;
        if (t >= 1) acc += (double)Dk[t] - (double)D0[t];
    }
    double incl = acc;  // inclusive prefix over the threads: inside the wave by shuffles, across the four waves through LDS
    for (int o = 1; o < 64; o <<= 1) {
        const double y = __shfl_up(incl, o);
        if ((tid & 63) >= o) incl += y;
    }
    if ((tid & 63) == 63) sm_part[tid >> 6] = incl;
    __syncthreads();
    double before = incl - acc;  // the sum over the runs of the threads below, i.e. over the columns above hi
    for (int w = 0; w < (tid >> 6); w++) before += sm_part[w];
    acc = before;
    for (int i = 0; i < run; i++) {
        const int t = hi - i;  // delta[t] excludes column t itself
        if (t >= 0 && t <= n - 1) sm_delta[t] = acc;
        if (t >= 1) acc += (double)Dk[t] - (double)D0[t];
    }
    __syncthreads();
    const int TS = T + 2, cells = NLP * TS;
    for (int base = tid; base < cells; base += 4 * 256) {
        float r[4], f0[4], f1[4];
        size_t o[4];
        int sc[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = base + u * 256, g = i / TS, s = i - g * TS, a_id = NLP * k + g;
            const bool ok = i < cells && a_id < mc && s <= n - 1;
            sc[u] = ok ? s : -1;
            o[u] = (size_t)(ok ? a_id : NLP * k) * TS + (ok ? s : 0);
            r[u] = av.SR[o[u]];
            f0[u] = av.F0[o[u]];
            f1[u] = av.F1[o[u]];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int s = sc[u];
            if (s >= 0 && s <= n - 2) av.SR[o[u]] = (float)((double)r[u] + sm_delta[s]);
            if (s >= 1) {
                av.F0[o[u]] = (float)((double)f0[u] + sm_delta[s - 1]);
                av.F1[o[u]] = (float)((double)f1[u] + sm_delta[s - 1]);
            }
        }
    }
}

// Grid (CL-1, B).  Dynamic LDS: T+2 doubles.
__global__ __launch_bounds__(256) void pipeline_rebase_kernel(float *__restrict__ aux, const int64_t *__restrict__ out_len,
                                                             const int64_t *__restrict__ tgt_len, int L, int T, int Mc) {
    extern __shared__ double sm_dyn[];
    pipeline_rebase_block((int)blockIdx.x + 1, (int)blockIdx.y, aux, out_len, tgt_len, L, T, Mc, sm_dyn);
}

// After the sweeps side by side and the forward's redo: grid (2 CL - 1, B); the first CL-1 blocks of a sentence rebase the
// forward tables, the other CL finish the outside sweep's.  Dynamic LDS: 2 (T+4) doubles.
__global__ __launch_bounds__(256) void pipeline_finish_kernel(float *__restrict__ aux, const int64_t *__restrict__ out_len,
                                                             const int64_t *__restrict__ tgt_len, int L, int T, int Mc, int CL,
                                                             float *__restrict__ S) {
    extern __shared__ double sm_dyn[];
    // a sentence whose second chance was given up (see inside_redo_ml1_stream_kernel) becomes an invalid one
    if (blockIdx.x == 0 && threadIdx.x == 0 && ExchangeView(aux, blockIdx.y, Mc, T).flags[FLAG_GIVEN_UP] != 0)
        S[(size_t)blockIdx.y * Mc * (T + 2)] = __builtin_nanf("");
    if ((int)blockIdx.x < CL - 1)  // workgroup-uniform
        pipeline_rebase_block((int)blockIdx.x + 1, (int)blockIdx.y, aux, out_len, tgt_len, L, T, Mc, sm_dyn);
    else
        pipeline_finish_outside_block((int)blockIdx.x - (CL - 1), (int)blockIdx.y, aux, out_len, tgt_len, L, T, Mc, sm_dyn);
}

// Outside sweep of one block.  Same tables as inside_bwd_ml1_stream_kernel.  Dynamic LDS: D [T+4], then (MATCH_LDS) the
// emissions of the block's nodes, main [NLP][T] and leaf [NLP][T].
template <int NQ, bool MATCH_LDS>
__global__ __launch_bounds__(NTP) void inside_bwd_ml1_pipe_kernel(const float *__restrict__ S, float *__restrict__ aux,
                                                                 const float *__restrict__ match_all,
                                                                 const int64_t *__restrict__ out_len,
                                                                 const int64_t *__restrict__ tgt_len, int L, int T, int Mc,
                                                                 int spin_limit) {
    constexpr int MP = 64 * NQ, CL = MP / NLP;
    __shared__ __attribute__((aligned(16))) float w0[2][MP];
    __shared__ __attribute__((aligned(16))) float w1[2][MP];
    __shared__ int sm_dead;
    extern __shared__ float sm_D[];  // [T+4]
    float *sm_main = sm_D + (T + 4), *sm_leaf = sm_main + NLP * T;
    const int b = blockIdx.x / CL, k = blockIdx.x % CL;  // the leading (lowest) block first
    const int tid = threadIdx.x, gidx = (tid >> 4) & (NLP - 1), j = tid & 15, lane = tid & 63;
    const bool collector = tid >= 16 * NLP;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *mt = match_all + (size_t)b * L * T;
    const float *Sb = S + (size_t)b * Mc * (T + 2);
    AuxViewStream av(aux, b, Mc, T);
    ExchangeView xv(aux, b, Mc, T);
    const float ll = Sb[0];
    const bool valid = lengths_ok(m, n, L, T) && (ll == ll) && (fabsf(ll) != __builtin_huge_valf());
    if (!valid) return;  // the posterior kernels write zeros for such sentences
    const int mc = m / 2;
    if (NLP * k >= mc) return;  // no node of the sentence in this block: nobody waits for it
    for (int i = tid; i < T + 4; i += NTP) sm_D[i] = av.D[i];
    for (int i = tid; i < 2 * MP; i += NTP) {
        (&w0[0][0])[i] = NEG_INF_F;
        (&w1[0][0])[i] = NEG_INF_F;
    }
    if (tid == 0) sm_dead = 0;
    if (MATCH_LDS) {
        for (int i = tid; i < NLP * T; i += NTP) {
            const int g = i / T, s = i - g * T, node = NLP * k + g;
            const bool ok = node < mc && s < n;
            sm_main[i] = ok ? to_b2(mt[(size_t)(2 * node + 1) * T + s]) : NEG_INF_F;
            sm_leaf[i] = (ok && node >= 1) ? to_b2(mt[(size_t)(2 * node) * T + s]) : NEG_INF_F;
        }
    }

    // this lane's node and its transposed link rows: parents a <= c, chunks [0, q1)
    const int c_id = NLP * k + gidx;
    const bool live = c_id < mc;
    const int ci = live ? c_id : NLP * k;
    const int q1 = (NLP * k + NLP - 1) / 64 + 1;
    float4 A0[NQ], A1[NQ];
    if (!collector) {
        const float4 *r0 = reinterpret_cast<const float4 *>(av.At + ((size_t)0 * Mc + ci) * MP) + j;
        const float4 *r1 = reinterpret_cast<const float4 *>(av.At + ((size_t)1 * Mc + ci) * MP) + j;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            A0[q] = r0[16 * q];
            A1[q] = r1[16 * q];
        }
    }
    const float *ra = mt + (size_t)(2 * ci + 1) * T, *rl = mt + (size_t)(2 * ci) * T;
    __syncthreads();  // sm_D, the cleared columns
    const float beta00 = -av.SR[0];  // relative to the offset of column 0
    const float w00 = (to_b2(mt[(size_t)1 * T]) + beta00) - sm_D[1];
    if (tid == 0) w0[1][0] = w00;
    float bp = (c_id == 0) ? beta00 : NEG_INF_F;  // the node's outside score one column earlier
    if (!collector && j == 0 && live) {
        av.BETA[(size_t)c_id * (T + 2)] = bp;
        av.W0[(size_t)c_id * (T + 2) + 1] = (c_id == 0) ? w00 : NEG_INF_F;
        av.W1[(size_t)c_id * (T + 2) + 1] = NEG_INF_F;
    }
    float mc_t, ml_p;  // main[c][t], leaf[c][t-1]
    if (MATCH_LDS) {
        mc_t = sm_main[gidx * T + 1];
        ml_p = sm_leaf[gidx * T];
    } else {
        mc_t = live ? to_b2(ra[1]) : NEG_INF_F;
        ml_p = (live && ci >= 1) ? to_b2(rl[0]) : NEG_INF_F;
    }
    // The link rows must have arrived before the sweep starts: a wait for them inside the loop would, from the second
    // column on, be a wait for the stores of the column before.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    unsigned *Xb = xv.bw;
    unsigned x0[NQ], x1[NQ];  // collector: the entries of the blocks below, requested one step before they are handed on
#pragma unroll
    for (int r = 0; r < NQ; r++) {
        const bool need = collector && k > 0 && n >= 3;
        x0[r] = need ? entry_load(Xb + (size_t)2 * 2 * MP + 64 * r + lane) : __float_as_uint(NEG_INF_F);
        x1[r] = need ? entry_load(Xb + (size_t)2 * 2 * MP + MP + 64 * r + lane) : __float_as_uint(NEG_INF_F);
    }
    for (int t = 1; t <= n - 1; t++) {
        const float *c0 = w0[t & 1], *c1 = w1[t & 1];
        float *n0 = w0[(t + 1) & 1], *n1 = w1[(t + 1) & 1];
        const bool more = t < n - 1;
        if (collector) {
            if (more && k > 0) {  // the weights of the blocks below for column t+1, requested one iteration ago
                const unsigned *src = Xb + (size_t)(t + 1) * 2 * MP + lane;
                // the requests went out for every lane (a branch around a load ends in a wait for it); entries of other
                // blocks' nodes beyond the sentence are never written and read as -inf
#pragma unroll
                for (int r = 0; r < NQ; r++) {
                    if (64 * r + lane >= min(NLP * k, mc)) {
                        x0[r] = __float_as_uint(NEG_INF_F);
                        x1[r] = __float_as_uint(NEG_INF_F);
                    }
                }
                for (int spins = 0;; spins++) {
                    bool pending = false;
#pragma unroll
                    for (int r = 0; r < NQ; r++) pending |= (x0[r] == EMPTY32) | (x1[r] == EMPTY32);
                    if (!__any(pending)) break;
                    if (spins >= spin_limit || ((spins & 63) == 63 && gave_up(xv.flags + FLAG_BWD))) {
                        sm_dead = 1;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(2);  // leave the issue slots of this SIMD to its compute wave
#pragma unroll
                    for (int r = 0; r < NQ; r++) {
                        if (x0[r] == EMPTY32) x0[r] = entry_load(src + 64 * r);
                        if (x1[r] == EMPTY32) x1[r] = entry_load(src + MP + 64 * r);
                    }
                }
#pragma unroll
                for (int r = 0; r < NQ; r++) {
                    const int i = 64 * r + lane;
                    if (i < NLP * k) {
                        n0[i] = (x0[r] == EMPTY32) ? NEG_INF_F : __uint_as_float(x0[r]);
                        n1[i] = (x1[r] == EMPTY32) ? NEG_INF_F : __uint_as_float(x1[r]);
                    }
                }
            }
            if (t + 2 <= n - 1 && k > 0) {  // request column t+2 now: it has the whole next step to arrive
                const unsigned *src = Xb + (size_t)(t + 2) * 2 * MP + lane;
#pragma unroll
                for (int r = 0; r < NQ; r++) {
                    x0[r] = entry_load(src + 64 * r);
                    x1[r] = entry_load(src + MP + 64 * r);
                }
            }
        } else {
            const float d_next = sm_D[t + 1], d_both = d_next + sm_D[t];
            float mc_raw = 0.f, ml_raw = 0.f;
            if (more) {
                mc_raw = MATCH_LDS ? sm_main[gidx * T + t + 1] : ra[t + 1];
                ml_raw = MATCH_LDS ? sm_leaf[gidx * T + t] : rl[t];
            }
            const float4 *u0 = reinterpret_cast<const float4 *>(c0) + j, *u1 = reinterpret_cast<const float4 *>(c1) + j;
            float beta, unused;
            slab_row_lse<NQ, true>(A0, A1, u0, u1, 0, q1, live, true, bp, beta, unused);
            if (!live) beta = NEG_INF_F;
            const float nw0 = (mc_t + beta) - d_next;
            const float nw1 = ((ml_p + mc_t) + bp) - d_both;
            if (j == 0) {
                n0[c_id] = nw0;
                n1[c_id] = nw1;
                if (live) {
                    if (more) {
                        entry_store(Xb + (size_t)(t + 1) * 2 * MP + c_id, nw0);
                        entry_store(Xb + (size_t)(t + 1) * 2 * MP + MP + c_id, nw1);
                    }
                    av.BETA[(size_t)c_id * (T + 2) + t] = beta;
                    av.W0[(size_t)c_id * (T + 2) + t + 1] = nw0;
                    av.W1[(size_t)c_id * (T + 2) + t + 1] = nw1;
                }
            }
            bp = beta;
            mc_t = MATCH_LDS ? mc_raw : (live ? to_b2(mc_raw) : NEG_INF_F);
            ml_p = MATCH_LDS ? ml_raw : ((live && ci >= 1) ? to_b2(ml_raw) : NEG_INF_F);
        }
        lds_barrier();
        if (sm_dead) {  // uniform: written before the barrier
            if (tid == 0) __hip_atomic_store(xv.flags + FLAG_BWD, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
}

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

__global__ void fill_zero_kernel(float *p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.f;
}


// loss = -(1/B) * sum_b [ll_b finite] ll_b / n_b and the number of invalid sentences (nat_pcfg_loss.py:123-135), reduced
// in a fixed order by one workgroup.  out[0] = loss, out[1] = invalid count.
__global__ __launch_bounds__(256) void criterion_loss_kernel(const float *__restrict__ S, const int64_t *__restrict__ tgt_len,
                                                            float *__restrict__ out, int B, int Mc, int T, float *__restrict__ ll_out) {
    criterion_loss_block<256>(LossTask{S, tgt_len, out, B, (int64_t)Mc * (T + 2), ll_out});
}

// The pipelined sweeps are used while a batch needs no more than g_pipeline_max_wg workgroups.  The default is no limit in
// practice: measured at 512 graph nodes and 140 target tokens they beat one workgroup per sentence 3.5x at 16 sentences
// and still 1.8x at 512 sentences (8192 workgroups: the blocks of a sentence are adjacent in dispatch order, leading
// block first, so a block never waits for one that has not been started).  Both numbers can be changed through
// pcfgnat_pipeline_config.
std::atomic<int> g_pipeline_max_wg{1 << 20}, g_pipeline_spin_limit{PCFGNAT_DEFAULT_SPIN_LIMIT};
std::atomic<int> g_pipeline_spin_limit_outside{-1};  // side-by-side launch only; negative: the common limit
// Bound of the one wait of the second-chance launch (the outside sweep's workgroup for the forward's, where both are
// redone), in polls of about a microsecond.  pcfgnat_pipeline_redo_wait_limit.
constexpr int DEFAULT_REDO_WAIT_LIMIT = 1 << 23;
std::atomic<int> g_redo_wait_limit{DEFAULT_REDO_WAIT_LIMIT};
// Largest base-2 exponent a factor of the rule posteriors of long graphs may have on the matrix cores (see
// links_grad_ml1_stream_kernel); a tile beyond it is recomputed term by term.  pcfgnat_links_grad_range_limit.
std::atomic<float> g_links_grad_range_limit{120.f};
// How a call sweeps its long graphs, decided once per call from one reading of the process-wide setting (a setting that
// changes while a call is being enqueued must not reach half of its launches).
struct PipelinePlan {
    int NQ;             // chunks of 64 nodes per sentence; 0: the pipelined sweeps do not apply
    bool side_by_side;  // forward and outside pipeline in one launch
};
PipelinePlan pipeline_plan(int B, int T, int Mc) {
    const int max_wg = g_pipeline_max_wg.load();
    const int NQ = stream_mp(Mc) / 64, CL = 64 * NQ / NLP;
    PipelinePlan plan{0, false};
    if (NQ >= 2 && NQ <= 8 && T + 2 < 4096 && (int64_t)B * CL <= max_wg) {
        plan.NQ = NQ;
        plan.side_by_side = (int64_t)2 * B * CL <= max_wg;
    }
    return plan;
}

template <int NQ>
int launch_fwd_pipe(const float *match_all, const int64_t *ol, const int64_t *tl, float *S, float *aux, int B, int L, int T, int Mc,
                    hipStream_t stream, bool both) {
    constexpr int CL = 64 * NQ / NLP;
    const size_t match_bytes = (size_t)2 * NLP * T * sizeof(float);
    if (both) {  // the outside pipeline in the same launch, behind the forward one in dispatch order
        const int spin_out = g_pipeline_spin_limit_outside.load() >= 0 ? g_pipeline_spin_limit_outside.load() : g_pipeline_spin_limit.load();
        // while every block of both pipelines can have a compute unit of its own: claim more than half of a unit's LDS so
        // that no two blocks share one (and its instruction issue), and spread the outside sweep's collecting over four waves
        const bool roomy = 2 * B * CL <= device_compute_units();
        if (match_bytes <= LDS_BUDGET - 8192) {
            const size_t lds = (roomy && match_bytes < PAD_EXCLUSIVE_LDS) ? PAD_EXCLUSIVE_LDS : match_bytes;
            if (roomy) {
                auto k = inside_both_ml1_pipe_kernel<NQ, true, 4>;
                PCFGNAT_DYNAMIC_LDS(k, lds);
                hipLaunchKernelGGL(k, dim3(2 * B * CL), dim3(16 * NLP + 256), lds, stream, match_all, ol, tl, S, aux, L, T, Mc,
                                   g_pipeline_spin_limit.load(), spin_out, B * CL);
            } else {
                auto k = inside_both_ml1_pipe_kernel<NQ, true, 1>;
                PCFGNAT_DYNAMIC_LDS(k, lds);
                hipLaunchKernelGGL(k, dim3(2 * B * CL), dim3(NTP), lds, stream, match_all, ol, tl, S, aux, L, T, Mc,
                                   g_pipeline_spin_limit.load(), spin_out, B * CL);
            }
        } else {
            hipLaunchKernelGGL((inside_both_ml1_pipe_kernel<NQ, false, 1>), dim3(2 * B * CL), dim3(NTP), 0, stream, match_all, ol, tl, S, aux,
                               L, T, Mc, g_pipeline_spin_limit.load(), spin_out, B * CL);
        }
    } else if (match_bytes <= LDS_BUDGET - 8192 && B * CL <= device_compute_units()) {  // a compute unit per block: four collector waves
        auto k = inside_fwd_ml1_pipe_kernel<NQ, true, 4>;
        const size_t lds = match_bytes < PAD_EXCLUSIVE_LDS ? PAD_EXCLUSIVE_LDS : match_bytes;
        PCFGNAT_DYNAMIC_LDS(k, lds);
        hipLaunchKernelGGL(k, dim3(B * CL), dim3(16 * NLP + 256), lds, stream, match_all, ol, tl, S, aux, L, T, Mc,
                           g_pipeline_spin_limit.load());
    } else if (match_bytes <= LDS_BUDGET - 8192) {
        auto k = inside_fwd_ml1_pipe_kernel<NQ, true>;
        PCFGNAT_DYNAMIC_LDS(k, match_bytes);
        hipLaunchKernelGGL(k, dim3(B * CL), dim3(NTP), match_bytes, stream, match_all, ol, tl, S, aux, L, T, Mc,
                           g_pipeline_spin_limit.load());
    } else {
        hipLaunchKernelGGL((inside_fwd_ml1_pipe_kernel<NQ, false>), dim3(B * CL), dim3(NTP), 0, stream, match_all, ol, tl, S, aux, L, T,
                           Mc, g_pipeline_spin_limit.load());
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    if (both) return PCFGNAT_OK;  // rebased together with the outside tables, once the redo of the forward has run
    hipLaunchKernelGGL(pipeline_rebase_kernel, dim3(CL - 1, B), dim3(256), (size_t)(T + 2) * sizeof(double), stream, aux, ol, tl, L, T,
                       Mc);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
template <int NQ>
int launch_bwd_pipe(const float *S, float *aux, const float *match_all, const int64_t *ol, const int64_t *tl, int B, int L, int T,
                    int Mc, hipStream_t stream) {
    constexpr int CL = 64 * NQ / NLP;
    const size_t base = (size_t)(T + 4) * sizeof(float), with_match = base + (size_t)2 * NLP * T * sizeof(float);
    if (with_match <= LDS_BUDGET - 8192) {
        auto k = inside_bwd_ml1_pipe_kernel<NQ, true>;
        PCFGNAT_DYNAMIC_LDS(k, with_match);
        hipLaunchKernelGGL(k, dim3(B * CL), dim3(NTP), with_match, stream, S, aux, match_all, ol, tl, L, T, Mc,
                           g_pipeline_spin_limit.load());
    } else {
        hipLaunchKernelGGL((inside_bwd_ml1_pipe_kernel<NQ, false>), dim3(B * CL), dim3(NTP), base, stream, S, aux, match_all, ol, tl, L,
                           T, Mc, g_pipeline_spin_limit.load());
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// zero_slabs: links_grad, where the call also has the backward to do (its slab is then zeroed here, beside the compact copies)
int launch_fwd_stream(const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux, int B,
                      int L, int T, int Mc, hipStream_t stream, int NQ, bool side_by_side = false, float *zero_slabs = nullptr) {
    const int MP = stream_mp(Mc);
    PCFGNAT_REQUIRE(((uintptr_t)aux & 15) == 0, "pcfg_loss: aux must be 16-byte aligned");
    hipLaunchKernelGGL(compact_links_ml1_kernel, dim3(MP / 32, MP / 32, B), dim3(256), 0, stream, links, ol, aux, L, T, Mc, MP, zero_slabs);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    // pipelined sweep first where it applies; the one-workgroup sweep then only redoes sentences whose blocks gave up
    int rc = PCFGNAT_OK;
    switch (NQ) {
        case 2: rc = launch_fwd_pipe<2>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 3: rc = launch_fwd_pipe<3>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 4: rc = launch_fwd_pipe<4>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 5: rc = launch_fwd_pipe<5>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 6: rc = launch_fwd_pipe<6>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 7: rc = launch_fwd_pipe<7>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 8: rc = launch_fwd_pipe<8>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        default: break;
    }
    if (rc != PCFGNAT_OK) return rc;
    const int only_flagged = NQ != 0;
    const size_t base = ((size_t)4 * MP + 32) * sizeof(float);
    const size_t with_match = base + (size_t)2 * Mc * T * sizeof(float);
    if (side_by_side) {
        // both pipelines have run: one launch for the second chance of either sweep (in the normal case it finds no flag
        // set and ends at once), then both sweeps' tables to common offsets and the corrections of the posteriors
        const size_t base_bwd = ((size_t)5 * MP + T + 4) * sizeof(float);
        const size_t lds = base > base_bwd ? base : base_bwd;
        const int WAIT_LIMIT = g_redo_wait_limit.load();  // polls of about a microsecond
        if (Mc <= NT / 4)
            hipLaunchKernelGGL(inside_redo_ml1_stream_kernel<4>, dim3(B, 2), dim3(NT), lds, stream, match_all, links, ol, tl, S, aux, L, T,
                               Mc, MP, WAIT_LIMIT);
        else
            hipLaunchKernelGGL(inside_redo_ml1_stream_kernel<8>, dim3(B, 2), dim3(NT), lds, stream, match_all, links, ol, tl, S, aux, L, T,
                               Mc, MP, WAIT_LIMIT);
        PCFGNAT_HIP_CHECK(hipGetLastError());
        const int CL = 64 * NQ / NLP;
        hipLaunchKernelGGL(pipeline_finish_kernel, dim3(2 * CL - 1, B), dim3(256), (size_t)2 * (T + 4) * sizeof(double), stream, aux, ol, tl,
                           L, T, Mc, CL, S);
        PCFGNAT_HIP_CHECK(hipGetLastError());
        return PCFGNAT_OK;
    }
    if (with_match <= LDS_BUDGET) {
        auto k = inside_fwd_ml1_stream_kernel<true, 4>;
        PCFGNAT_DYNAMIC_LDS(k, with_match);
        hipLaunchKernelGGL(k, dim3(B), dim3(NT), with_match, stream, match_all, links, ol, tl, S, aux, L, T, Mc, MP, only_flagged);
    } else {
        hipLaunchKernelGGL((inside_fwd_ml1_stream_kernel<false, 4>), dim3(B), dim3(NT), base, stream, match_all, links, ol, tl, S, aux, L,
                           T, Mc, MP, only_flagged);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// side_by_side: the outside pipeline has already run, beside the forward one (launch_both_stream): only the redo of the
// sentences it gave up and the posteriors (with their per-column corrections) are left to do.
int launch_bwd_stream(const float *go, const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol,
                      const int64_t *tl, float *mg, float *lg, int B, int L, int T, int Mc, Seed seed, hipStream_t stream, int NQ,
                      bool side_by_side = false, bool slabs_zeroed = false) {
    const int MP = stream_mp(Mc);
    const int tiles = (Mc + LG_TILE - 1) / LG_TILE;
    PCFGNAT_REQUIRE(((uintptr_t)aux & 15) == 0, "pcfg_loss_backward: aux must be 16-byte aligned");
    const size_t base = ((size_t)5 * MP + T + 4) * sizeof(float);
    const size_t with_match = base + (size_t)2 * Mc * T * sizeof(float);
    int rc = PCFGNAT_OK;
    switch (side_by_side ? 0 : NQ) {
        case 2: rc = launch_bwd_pipe<2>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 3: rc = launch_bwd_pipe<3>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 4: rc = launch_bwd_pipe<4>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 5: rc = launch_bwd_pipe<5>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 6: rc = launch_bwd_pipe<6>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 7: rc = launch_bwd_pipe<7>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 8: rc = launch_bwd_pipe<8>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        default: break;
    }
    if (rc != PCFGNAT_OK) return rc;
    const int only_flagged = NQ != 0;
    // lanes per node: four while one pass covers all nodes; beyond that the outside sweep measured faster with eight
    if (side_by_side) {
        // (the outside sweep's second chance has run in the launch it shares with the forward's: launch_fwd_stream)
    } else if (with_match <= LDS_BUDGET) {
        auto k = Mc <= NT / 4 ? inside_bwd_ml1_stream_kernel<true, 4> : inside_bwd_ml1_stream_kernel<true, 8>;
        PCFGNAT_DYNAMIC_LDS(k, with_match);
        hipLaunchKernelGGL(k, dim3(B), dim3(NT), with_match, stream, S, aux, match_all, ol, tl, L, T, Mc, MP, only_flagged);
    } else {
        auto k = Mc <= NT / 4 ? inside_bwd_ml1_stream_kernel<false, 4> : inside_bwd_ml1_stream_kernel<false, 8>;
        hipLaunchKernelGGL(k, dim3(B), dim3(NT), base, stream, S, aux, match_all, ol, tl, L, T, Mc, MP, only_flagged);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    if (!slabs_zeroed) {
        const size_t nlg = (size_t)B * L * 2 * L;
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, stream, lg, nlg);
        PCFGNAT_HIP_CHECK(hipGetLastError());
    }
    const int use_corr = side_by_side ? 1 : 0;
    bool small;
    const int span = links_grad_span(T, (long)B * tiles * (tiles + 1) / 2, small);
    auto lgk = small ? links_grad_ml1_stream_kernel<LG_SPAN_SMALL / 32> : links_grad_ml1_stream_kernel<LG_SPAN / 32>;
    PCFGNAT_DYNAMIC_LDS(lgk, links_grad_lds_bytes(span));
    // The workgroups below the diagonal of the tile grid have no rules to do: they take the emission posteriors while that
    // leaves each of their threads a handful of cells; otherwise those get a launch of their own.
    const long spare_threads = (long)tiles * (tiles - 1) / 2 * 256;
    const bool emis_inside = spare_threads > 0 && (long)L * T <= 16 * spare_threads;
    hipLaunchKernelGGL(lgk, dim3(tiles, tiles, B), dim3(256), links_grad_lds_bytes(span), stream, go, S, aux, links, ol, tl, lg, L, T,
                       Mc, seed, use_corr, g_links_grad_range_limit.load(), span,
                       MatchGradArgs{match_all, emis_inside ? mg : nullptr});
    PCFGNAT_HIP_CHECK(hipGetLastError());
    if (!emis_inside) {
        hipLaunchKernelGGL(match_grad_ml1_stream_kernel, dim3((L * T + 255) / 256, B), dim3(256), 0, stream, go, S, aux, match_all, ol, tl,
                           mg, L, T, Mc, seed, use_corr);
        PCFGNAT_HIP_CHECK(hipGetLastError());
    }
    return PCFGNAT_OK;
}

template <int R>
int launch_fwd(const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux, int B, int L,
               int T, int Mc, hipStream_t stream) {
    const size_t base = ((size_t)head_floats(T) + 2 * 64 * R) * sizeof(float);
    const size_t with_tab = base + ((size_t)2 * Mc * T + (size_t)3 * Mc * (T + 2)) * sizeof(float);
    if (with_tab <= LDS_BUDGET) {
        auto k = inside_fwd_ml1_kernel<R, true>;
        PCFGNAT_DYNAMIC_LDS(k, with_tab);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), with_tab, stream, match_all, links, ol, tl, S, aux, L, T, Mc);
    } else {
        auto k = inside_fwd_ml1_kernel<R, false>;
        PCFGNAT_REQUIRE(base <= LDS_BUDGET, "pcfg_loss: target length %d too large for the column offsets in LDS", T);
        PCFGNAT_DYNAMIC_LDS(k, base);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), base, stream, match_all, links, ol, tl, S, aux, L, T, Mc);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

template <int R>
int launch_bwd(const float *go, const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol,
               const int64_t *tl, float *mg, float *lg, int B, int L, int T, int Mc, Seed seed, hipStream_t stream) {
    const size_t base = ((size_t)head_floats(T) + 4 * 64 * R) * sizeof(float);
    const size_t with_tab = base + ((size_t)2 * Mc * T + (size_t)4 * Mc * (T + 2)) * sizeof(float);
    if (with_tab <= LDS_BUDGET) {
        auto k = inside_bwd_ml1_kernel<R, true>;
        PCFGNAT_DYNAMIC_LDS(k, with_tab);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), with_tab, stream, go, S, aux, match_all, links, ol, tl, mg, lg, L, T, Mc, seed);
    } else {
        auto k = inside_bwd_ml1_kernel<R, false>;
        PCFGNAT_REQUIRE(base <= LDS_BUDGET, "pcfg_loss_backward: target length %d too large for the column offsets in LDS", T);
        PCFGNAT_DYNAMIC_LDS(k, base);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), base, stream, go, S, aux, match_all, links, ol, tl, mg, lg, L, T, Mc, seed);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// Returns PCFGNAT_EUNSUPPORTED (without a message being an error for the caller) when the fused kernel does not apply.
template <int R>
int launch_fused(const float *go, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux,
                 float *mg, float *lg, int B, int L, int T, int Mc, Seed seed, hipStream_t stream, bool *done,
                 PadFill pad = PadFill{nullptr, 0}, bool *pad_done = nullptr) {
    const size_t need = ((size_t)head_floats(T) + 4 * 64 * R + (size_t)4 * Mc * (T + 2) + (size_t)2 * Mc * T) * sizeof(float);
    *done = false;
    if (R == 1) {  // the two sweeps side by side as two workgroups per sentence, then the posteriors
        const size_t fwd_bytes = ((size_t)head_floats(T) + 2 * 64 + (size_t)2 * Mc * T + (size_t)3 * Mc * (T + 2)) * sizeof(float);
        const size_t pair_bytes = fwd_bytes > outside_role_bytes(Mc, T) ? fwd_bytes : outside_role_bytes(Mc, T);
        const size_t comb_bytes = ((size_t)(T + 4) + (size_t)Mc * (T + 2) + (size_t)8 * (T + 2)) * sizeof(float);
        if (pair_bytes <= LDS_BUDGET && comb_bytes <= 64 * 1024 && L <= 128) {
            PCFGNAT_REQUIRE(((uintptr_t)aux & 7) == 0, "pcfg_loss_forward_backward: aux must be 8-byte aligned");
            PCFGNAT_DYNAMIC_LDS(inside_pair_ml1_kernel, pair_bytes);
            // the fill rides along only while the sweeps leave compute units free for it (the gather backward writes the
            // zeros itself otherwise)
            const bool fill = pad.base != nullptr && pad.row_bytes > 0 && 2 * B <= pad_max_sweep_wgs();
            // With the fill, every workgroup of the launch claims more than half of a compute unit's LDS, so that no fill
            // workgroup shares a compute unit (and its instruction issue) with a sweep.
            const size_t launch_bytes = (fill && pair_bytes < PAD_EXCLUSIVE_LDS) ? PAD_EXCLUSIVE_LDS : pair_bytes;
            if (launch_bytes != pair_bytes)
                PCFGNAT_DYNAMIC_LDS(inside_pair_ml1_kernel, launch_bytes);
            hipLaunchKernelGGL(inside_pair_ml1_kernel, dim3((2 + (fill ? PAD_WGS : 0)) * B), dim3(NTR), launch_bytes, stream, match_all,
                               links, ol, tl, S, aux, L, T, Mc, B, pad);
            PCFGNAT_HIP_CHECK(hipGetLastError());
            if (fill && pad_done) *pad_done = true;
            hipLaunchKernelGGL(inside_combine_ml1_kernel, dim3(16, B), dim3(256), comb_bytes, stream, go, S, aux, match_all, links, ol, tl,
                               mg, lg, L, T, Mc, seed);
            PCFGNAT_HIP_CHECK(hipGetLastError());
            *done = true;
            return PCFGNAT_OK;
        }
    }
    if (need > LDS_BUDGET) return PCFGNAT_OK;
    auto k = inside_fused_ml1_kernel<R>;
    PCFGNAT_DYNAMIC_LDS(k, need);
    hipLaunchKernelGGL(k, dim3(B), dim3(NTR), need, stream, go, match_all, links, ol, tl, S, mg, lg, L, T, Mc, seed);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    *done = true;
    return PCFGNAT_OK;
}

int check_dims(const char *who, int64_t B, int64_t L, int64_t T, int64_t ml) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 4 && T >= 2, "%s: need B >= 0, L >= 4, T >= 2 (got B=%lld L=%lld T=%lld)", who, (long long)B,
                    (long long)L, (long long)T);
    PCFGNAT_REQUIRE(ml >= 0, "%s: links must have at least one left option", who);
    PCFGNAT_REQUIRE(L <= 4096 && T <= 4096 && B <= 65535, "%s: dimension too large (L, T <= 4096, B <= 65535)", who);
    PCFGNAT_REQUIRE(ml <= 63 && L >= ml + 3, "%s: max_left = %lld needs a graph of at least max_left + 3 nodes (and max_left <= 63)", who,
                    (long long)ml);
    return PCFGNAT_OK;
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

int pcfgnat::pipeline_max_workgroups() { return g_pipeline_max_wg.load(); }
int pcfgnat::pipeline_spin_limit() { return g_pipeline_spin_limit.load(); }

extern "C" void pcfgnat_pipeline_config(int max_workgroups, int spin_limit) {
    if (max_workgroups >= 0) g_pipeline_max_wg.store(max_workgroups);
    if (spin_limit >= 0) g_pipeline_spin_limit.store(spin_limit);
}

extern "C" void pcfgnat_pipeline_outside_spin_limit(int spin_limit) { g_pipeline_spin_limit_outside.store(spin_limit); }

extern "C" void pcfgnat_links_grad_range_limit(float log2_limit) { g_links_grad_range_limit.store(log2_limit); }

extern "C" void pcfgnat_pipeline_redo_wait_limit(int polls) { g_redo_wait_limit.store(polls < 0 ? DEFAULT_REDO_WAIT_LIMIT : polls); }

extern "C" int pcfgnat_pipeline_redo_counts(unsigned long long *inside_sweeps, unsigned long long *viterbi_sentences,
                                            unsigned long long *inside_given_up, int reset) {
    PCFGNAT_REQUIRE(inside_sweeps && viterbi_sentences && inside_given_up, "pipeline_redo_counts: null pointer");
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(inside_sweeps, HIP_SYMBOL(g_inside_redone), sizeof(*inside_sweeps)));
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(inside_given_up, HIP_SYMBOL(g_inside_given_up), sizeof(*inside_given_up)));
    if (reset) {
        const unsigned long long zero = 0;
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_inside_redone), &zero, sizeof(zero)));
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_inside_given_up), &zero, sizeof(zero)));
    }
    return viterbi_redo_count(viterbi_sentences, reset);
}

extern "C" size_t pcfgnat_pcfg_aux_floats(int64_t B, int64_t L, int64_t T, int64_t ml) {
    if (B <= 0 || L < 2 || T < 0 || ml < 0) return 0;
    if (ml != 1) return generic_aux_floats(B, L, T, ml);
    const int64_t Mc = (L - 2) / (ml + 1) + 1;
    if (Mc <= 64) return (size_t)B * aux_stride_reg((int)Mc, (int)T);
    return (size_t)B * aux_stride_stream((int)Mc, (int)T);
}

extern "C" int pcfgnat_pcfg_loss(const float *match_all, const float *links, const int64_t *output_length,
                                 const int64_t *target_length, float *S, float *aux, int64_t B, int64_t L, int64_t T, int64_t ml,
                                 void *stream) {
    int rc = check_dims("pcfg_loss", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(match_all && links && output_length && target_length && S && aux, "pcfg_loss: null pointer");
    if (ml != 1) return generic_forward(match_all, links, output_length, target_length, S, aux, B, L, T, ml, stream);
    const int Mc = (int)((L - 2) / 2 + 1);
    hipStream_t s = (hipStream_t)stream;
    if (Mc <= 64) return launch_fwd<1>(match_all, links, output_length, target_length, S, aux, (int)B, (int)L, (int)T, Mc, s);
    return launch_fwd_stream(match_all, links, output_length, target_length, S, aux, (int)B, (int)L, (int)T, Mc, s,
                             pipeline_plan((int)B, (int)T, Mc).NQ);
}

int pcfgnat::inside_backward_impl(const float *grad_output, const float *S, float *aux, const float *match_all, const float *links,
                                  const int64_t *output_length, const int64_t *target_length, float *match_all_grad, float *links_grad,
                                  int64_t B, int64_t L, int64_t T, int64_t ml, Seed seed, void *stream) {
    int rc = check_dims("pcfg_loss_backward", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(S && aux && match_all && links && output_length && target_length && match_all_grad && links_grad,
                    "pcfg_loss_backward: null pointer");
    if (ml != 1)
        return generic_backward(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T,
                                ml, seed, stream);
    const int Mc = (int)((L - 2) / 2 + 1);
    hipStream_t s = (hipStream_t)stream;
    if (Mc <= 64)
        return launch_bwd<1>(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, (int)B,
                             (int)L, (int)T, Mc, seed, s);
    return launch_bwd_stream(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, (int)B,
                             (int)L, (int)T, Mc, seed, s, pipeline_plan((int)B, (int)T, Mc).NQ);
}

extern "C" int pcfgnat_pcfg_loss_backward(const float *grad_output, const float *S, float *aux, const float *match_all,
                                          const float *links, const int64_t *output_length, const int64_t *target_length,
                                          float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                          void *stream) {
    return inside_backward_impl(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T,
                                ml, seed_of(B), stream);
}

int pcfgnat::inside_forward_backward_impl(const float *grad_output, const float *match_all, const float *links,
                                          const int64_t *output_length, const int64_t *target_length, float *S, float *aux,
                                          float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                          Seed seed, void *stream, PadFill pad, bool *pad_done) {
    if (pad_done) *pad_done = false;
    int rc = check_dims("pcfg_loss_forward_backward", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(match_all && links && output_length && target_length && S && aux && match_all_grad && links_grad,
                    "pcfg_loss_forward_backward: null pointer");
    const int Mc = (int)((L - 2) / 2 + 1);
    hipStream_t s = (hipStream_t)stream;
    bool done = false;
    if (ml != 1) {
        // general max_left: the two plain kernels
    } else if (Mc <= 64)
        rc = launch_fused<1>(grad_output, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad, (int)B, (int)L,
                             (int)T, Mc, seed, s, &done, pad, pad_done);
    if (rc != PCFGNAT_OK || done) return rc;
    const PipelinePlan plan = (ml == 1 && Mc > 64) ? pipeline_plan((int)B, (int)T, Mc) : PipelinePlan{0, false};
    if (plan.side_by_side) {  // the two pipelined sweeps in one launch
        rc = launch_fwd_stream(match_all, links, output_length, target_length, S, aux, (int)B, (int)L, (int)T, Mc, s, plan.NQ, true,
                               links_grad);
        if (rc != PCFGNAT_OK) return rc;
        return launch_bwd_stream(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, (int)B,
                                 (int)L, (int)T, Mc, seed, s, plan.NQ, true, true);
    }
    rc = pcfgnat_pcfg_loss(match_all, links, output_length, target_length, S, aux, B, L, T, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    return inside_backward_impl(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T,
                                ml, seed, stream);
}

extern "C" int pcfgnat_pcfg_loss_forward_backward(const float *grad_output, const float *match_all, const float *links,
                                                 const int64_t *output_length, const int64_t *target_length, float *S, float *aux,
                                                 float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T,
                                                 int64_t ml, void *stream) {
    return inside_forward_backward_impl(grad_output, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad,
                                        B, L, T, ml, seed_of(B), stream);
}

// ---------------------------------------------------------------------------------------------------------------
// pcfgnat_pcfg_loss_forward_backward for callers that cannot allocate device memory (code under HIP graph capture,
// serving loops, harnesses that forbid hipMalloc): the auxiliary table lives in a device array of fixed size that
// belongs to the library.  Every device the code object is loaded on holds its own copy of the array at its own
// address, looked up once per device; in host code the array's name is only a handle for that lookup, never an address.
// ---------------------------------------------------------------------------------------------------------------
namespace {
static __device__ __align__(256) float static_aux[PCFGNAT_STATIC_AUX_FLOATS];
constexpr int STATIC_AUX_MAX_DEVICES = 64;
float *g_static_aux_ptr[STATIC_AUX_MAX_DEVICES];
std::mutex g_static_aux_mutex;

// The address of the current device's copy of static_aux (looked up with that device current, kept for later calls).
int static_aux_address(float **out) {
    int dev = -1;
    PCFGNAT_HIP_CHECK(hipGetDevice(&dev));
    PCFGNAT_REQUIRE(dev >= 0 && dev < STATIC_AUX_MAX_DEVICES, "pcfg_loss_forward_backward_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_aux_mutex);
    if (g_static_aux_ptr[dev] == nullptr) {
        float *ptr = nullptr;
        PCFGNAT_HIP_CHECK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(static_aux)));
        if (ptr == nullptr) return pcfgnat::fail(PCFGNAT_EHIP, "pcfg_loss_forward_backward_static: no device address for the static table");
        g_static_aux_ptr[dev] = ptr;
    }
    *out = g_static_aux_ptr[dev];
    return PCFGNAT_OK;
}
}  // namespace

extern "C" size_t pcfgnat_static_aux_floats(void) { return (size_t)PCFGNAT_STATIC_AUX_FLOATS; }

extern "C" int pcfgnat_pcfg_loss_forward_backward_static(const float *grad_output, const float *match_all, const float *links,
                                                        const int64_t *output_length, const int64_t *target_length, float *S,
                                                        float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T,
                                                        int64_t ml, void *stream) {
    int rc = check_dims("pcfg_loss_forward_backward_static", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    const size_t need = pcfgnat_pcfg_aux_floats(B, L, T, ml);
    PCFGNAT_REQUIRE(need <= (size_t)PCFGNAT_STATIC_AUX_FLOATS,
                    "pcfg_loss_forward_backward_static: B=%lld L=%lld T=%lld max_left=%lld needs %zu floats of auxiliary table, the "
                    "library's static table holds %zu (use pcfgnat_pcfg_loss_forward_backward with a buffer of the caller's)",
                    (long long)B, (long long)L, (long long)T, (long long)ml, need, (size_t)PCFGNAT_STATIC_AUX_FLOATS);
    float *aux = nullptr;
    rc = static_aux_address(&aux);
    if (rc != PCFGNAT_OK) return rc;
    // every table the kernels read from aux is written earlier in the same call (arrival marks of the pipelined sweeps
    // included), so what an earlier call left in the array does not matter
    return inside_forward_backward_impl(grad_output, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad,
                                        B, L, T, ml, seed_of(B), stream);
}

int pcfgnat::criterion_loss_impl(const float *S, const int64_t *target_length, float *out, float *ll_out, int64_t B, int64_t L, int64_t T,
                                 int64_t ml, void *stream) {
    int rc = check_dims("criterion_loss", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_REQUIRE(B >= 1 && S && target_length && out, "criterion_loss: null pointer or empty batch");
    const int Mc = (int)((L - 2) / (ml + 1) + 1);
    hipLaunchKernelGGL(criterion_loss_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, S, target_length, out, (int)B, Mc, (int)T, ll_out);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_criterion_loss(const float *S, const int64_t *target_length, float *out, int64_t B, int64_t L, int64_t T,
                                      int64_t ml, void *stream) {
    return criterion_loss_impl(S, target_length, out, nullptr, B, L, T, ml, stream);
}

namespace pcfgnat {
// Best tree and the GLAT glue behind it in one launch (max_left = 1); glue.path receives the tree.
int best_tree_glue_ml1(const float *S, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, int64_t B,
                       int64_t L, int64_t T, const GlatGlueArgs &glue, void *stream) {
    const int Mc = (int)((L - 2) / 2 + 1);
    const size_t glue_bytes = ((size_t)3 * L + 2) * sizeof(float) + (size_t)T * sizeof(int64_t);
    size_t tables = (size_t)Mc * (T + 2) + (size_t)2 * Mc * T, with_links = tables + (size_t)2 * Mc * Mc;  // floats, rounded up to even
    tables += tables & 1;
    with_links += with_links & 1;
    PCFGNAT_REQUIRE(glue_bytes <= LDS_BUDGET, "glat_step: graph of %lld nodes too long", (long long)L);
#define PCFGNAT_TREE_GLUE(mode, floats)                                                                                               \
    do {                                                                                                                             \
        auto k = best_tree_glue_ml1_kernel<mode>;                                                                                    \
        const size_t lds = (size_t)(floats) * sizeof(float) + glue_bytes;                                                            \
        PCFGNAT_DYNAMIC_LDS(k, lds);                                                                                                 \
        hipLaunchKernelGGL(k, dim3((unsigned)B), dim3(BT_NT), lds, (hipStream_t)stream, S, match_all, links, ol, tl, (int)L, (int)T, Mc, \
                           (int)(floats), glue);                                                                                     \
    } while (0)
    if (with_links * sizeof(float) + glue_bytes <= LDS_BUDGET) PCFGNAT_TREE_GLUE(2, with_links);
    else if (tables * sizeof(float) + glue_bytes <= LDS_BUDGET) PCFGNAT_TREE_GLUE(1, tables);
    else PCFGNAT_TREE_GLUE(0, 0);
#undef PCFGNAT_TREE_GLUE
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
}  // namespace pcfgnat

extern "C" int pcfgnat_pcfg_best_tree(const float *S, float *aux, const float *match_all, const float *links,
                                      const int64_t *output_length, const int64_t *target_length, int64_t *tree, int64_t B, int64_t L,
                                      int64_t T, int64_t ml, void *stream) {
    int rc = check_dims("pcfg_best_tree", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(S && match_all && links && output_length && target_length && tree, "pcfg_best_tree: null pointer");
    if (ml != 1) {
        PCFGNAT_REQUIRE(aux != nullptr, "pcfg_best_tree: the auxiliary table of pcfg_loss is required for max_left != 1");
        return generic_best_tree(S, aux, match_all, links, output_length, target_length, tree, B, L, T, ml, stream);
    }
    const int Mc = (int)((L - 2) / 2 + 1);
    const size_t tables = ((size_t)Mc * (T + 2) + (size_t)2 * Mc * T) * sizeof(float);
    const size_t with_links = tables + (size_t)2 * Mc * Mc * sizeof(float);
    if (with_links <= LDS_BUDGET) {
        auto k = best_tree_ml1_kernel<2>;
        PCFGNAT_DYNAMIC_LDS(k, with_links);
        hipLaunchKernelGGL(k, dim3((unsigned)B), dim3(BT_NT), with_links, (hipStream_t)stream, S, match_all, links, output_length,
                           target_length, tree, (int)L, (int)T, Mc);
    } else if (tables <= LDS_BUDGET) {
        auto k = best_tree_ml1_kernel<1>;
        PCFGNAT_DYNAMIC_LDS(k, tables);
        hipLaunchKernelGGL(k, dim3((unsigned)B), dim3(BT_NT), tables, (hipStream_t)stream, S, match_all, links, output_length,
                           target_length, tree, (int)L, (int)T, Mc);
    } else {
        hipLaunchKernelGGL(best_tree_ml1_kernel<0>, dim3((unsigned)B), dim3(BT_NT), 0, (hipStream_t)stream, S, match_all, links,
                           output_length, target_length, tree, (int)L, (int)T, Mc);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
