// Pipelined sweeps of graphs of 130..1026 nodes: one workgroup per block of 16 main-chain nodes, the blocks of a sentence
// following each other through an exchange area in memory; forward, outside, both side by side, their second chance and
// the launch that brings every block's tables to common offsets.
// Part of inside.hip (one translation unit: the kernels share helpers and the anonymous namespace).
#pragma once
#include "inside_common.hip.h"

namespace pcfgnat {
namespace {

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
    // the column(s) first, all LDS reads in flight together: a read inside each chunk's branch (qa, qb are run-time values)
    // costs the block one LDS round trip per chunk and step
    float4 v0[NQ], v1[NQ];
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        v0[q] = u0[16 * q];
        if (JOINT) v1[q] = u1[16 * q];
    }
#pragma unroll
    for (int q = 0; q < NQ; q++) {  // (keeps the reads up here)
        asm volatile("" : "+v"(v0[q].x), "+v"(v0[q].y), "+v"(v0[q].z), "+v"(v0[q].w));
        if (JOINT) asm volatile("" : "+v"(v1[q].x), "+v"(v1[q].y), "+v"(v1[q].z), "+v"(v1[q].w));
    }
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        if (q >= qa && q < qb) {
            const float4 c0 = minus(v0[q], g);
            const float4 c1 = JOINT ? minus(v1[q], g) : c0;
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
                const float4 c0 = v0[q];
                const float4 c1 = JOINT ? v1[q] : c0;
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

}  // namespace
}  // namespace pcfgnat
