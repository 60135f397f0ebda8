// Shared pieces of the inside kernels (max_left = 1): the layout of the auxiliary table of graphs of up to 130 nodes,
// the column offsets all sweeps keep, the head of the sweeps' LDS.
// Part of inside.hip (one translation unit: the kernels share helpers and the anonymous namespace).
#pragma once
#include "common.hip.h"

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

}  // namespace
}  // namespace pcfgnat
