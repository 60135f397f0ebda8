// Inside loss and its exact backward for max_left = 3 (--left-tree-layer 2: up to three local nodes in front of every
// main-chain node), forward and backward in one launch, one workgroup per sentence.
//
// Replaces, for the inputs described below, the general loops of the reference's pcfg_loss.cu (:84-224, 262-349) and
// pcfg_loss_backward.cu (:28-603), which generic_ml.hip restates as they are.
//
// What the model can produce.  extract_links (models/glat_decomposed_with_link_two_hands_tri_pcfg.py:175) restricts right
// children to main-chain nodes, so a local node never has an allowed right child and its whole row of `links` is -inf.
// Without a finite rule of their own the local trees of pcfg_loss.cu:262-349 reduce to their leaves: of the three local
// nodes a-3, a-2, a-1 in front of main-chain node a only the two leaves (a-3 and a-1, the odd offsets of :288-300) carry
// anything, one token each.  The main-chain recursion (:148-214) then has three options per (parent a, right child c):
//     k = 0: no left child,        S[a][s] <- links[a,0,c] + match[a][s]                      + S[c][s+1]
//     k = 1: left child a-1,       S[a][s] <- links[a,1,c] + match[a-1][s] + match[a][s+1]    + S[c][s+2]
//     k = 3: left child a-3,       S[a][s] <- links[a,3,c] + match[a-3][s] + match[a][s+1]    + S[c][s+2]
// (k = 2, the inner local node a-2, has no table entry to contribute; the root a = 1 has no left option at all).
// A sentence qualifies when the twelve rules per group through which the reference's loops could build a composite local
// tree - links[x, k, c] for x in {a-3, a-2}, x < c < a, every k - are all -inf (NaN counts as -inf, as in :162); the
// kernel checks that itself and leaves every other sentence untouched for the plain kernels, launched behind it, which
// apply the same test and skip the sentences this kernel took (ml3_composite_rules below is the one predicate of both).
//
// Layout: 512 threads = 64 main-chain nodes x 8 lanes; a node's rules towards its right children (inside sweep) or from
// its parents (outside sweep) live in registers, eight children or parents per lane and left option; all tables in LDS
// as base-2 logarithms: S (inside), V = outside - inside, the row sums R_k[a][t] = log2 sum_c 2^(links[a,k,c] + S[c][t]),
// and the emissions of the main-chain nodes and of their two leaves.  One barrier per target position and sweep.  The
// gradients are posteriors: links_grad[a,k,c] = g * sum_t 2^(links + U_k[a][t] + S[c][t]), match_all_grad from the
// per-option masses q_k(a,s) = 2^(V[a][s] + emissions + R_k[a][s+j+1]).  Values are absolute (no per-column offsets):
// the kernel serves targets of up to 64 tokens, where float32 resolves the table entries to about 1e-5.
#include "common.hip.h"

namespace pcfgnat {
namespace {

constexpr int NT3 = 512;
constexpr int MC3_MAX = 64;  // main-chain nodes per sentence: graphs of up to 254 nodes
constexpr int T3_MAX = 64;
constexpr float LOG2E_F = 1.4426950408889634f;
constexpr float LN2_F = 0.6931471805599453f;

__device__ unsigned long long g_ml3_counts[2];  // diagnostic: sentences served by the kernel below, sentences left to the plain ones

__device__ __forceinline__ float g8_max(float v) {
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_ROW_HALF_MIRROR>(v));
    return v;
}
__device__ __forceinline__ float g8_sum(float v) {
    v += dpp_f<DPP_QUAD_XOR1>(v);
    v += dpp_f<DPP_QUAD_XOR2>(v);
    v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
    return v;
}
// log2 of the sum over the 8 lanes of a node of s * 2^m (s = 0 where m = -inf); every lane gets the result
__device__ __forceinline__ float g8_lse(float m, float s) {
    const float M = g8_max(m);
    float t = (m > NEG_INF_F) ? s * __builtin_amdgcn_exp2f(m - M) : 0.0f;
    t = g8_sum(t);
    return (M > NEG_INF_F) ? M + __builtin_amdgcn_logf(t) : NEG_INF_F;
}
__device__ __forceinline__ float log2_of(float x) { return (x == x) ? x * LOG2E_F : NEG_INF_F; }  // NaN terms count as -inf (:162)

struct Ml3Tables {
    float *S, *V, *R0, *R1, *R3, *M0, *M1, *M3;
    int TS;
    __device__ Ml3Tables(float *base, int Mc, int T) : TS(T + 3) {
        const size_t n = (size_t)Mc * TS;
        S = base, V = base + n, R0 = base + 2 * n, R1 = base + 3 * n, R3 = base + 4 * n, M0 = base + 5 * n, M1 = base + 6 * n,
        M3 = base + 7 * n;
    }
    __device__ int at(int a_id, int s) const { return a_id * TS + s; }
};

// NR: children (or parents) per lane, 8 NR >= the main-chain nodes of the padded graph
template <int NR>
__global__ __launch_bounds__(NT3) void inside_fused_ml3_kernel(const float *__restrict__ grad_out, const float *__restrict__ match_all,
                                                               const float *__restrict__ links_all, const int64_t *__restrict__ out_len,
                                                               const int64_t *__restrict__ tgt_len, float *__restrict__ S_all,
                                                               float *__restrict__ mg_all, float *__restrict__ lg_all, int L, int T, int Mc,
                                                               Seed seed) {
    extern __shared__ float lds[];
    __shared__ float s_u[2][3][MC3_MAX];
    const int b = blockIdx.x, tid = threadIdx.x, g = tid >> 3, l = tid & 7;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const float *match = match_all + (size_t)b * L * T;
    const float *links = links_all + (size_t)b * L * 4 * L;
    const int TS_out = T + 2;
    float *S_out = S_all + (size_t)b * Mc * TS_out;
    float *mg = mg_all + (size_t)b * L * T;
    float *lg = lg_all + (size_t)b * L * 4 * L;
    const bool lengths_ok = m >= 6 && m <= L && ((m - 2) & 3) == 0 && n >= 2 && n <= T;
    const bool composite = lengths_ok && ml3_composite_rules<NT3>(links, L, m, tid);
    if (tid == 0) atomicAdd(&g_ml3_counts[composite ? 1 : 0], 1ULL);
    if (composite) return;  // the plain kernels take this sentence

    if (!lengths_ok) {  // outside the contract: NaN log-likelihood, zero gradients
        for (int i = tid; i < Mc * TS_out; i += NT3) S_out[i] = (i == 0) ? __builtin_nanf("") : NEG_INF_F;
        for (int i = tid; i < L * T; i += NT3) mg[i] = 0.0f;
        for (int i = tid; i < 4 * L * L; i += NT3) lg[i] = 0.0f;
        return;
    }
    const Ml3Tables tb(lds, Mc, T);
    const int TS = tb.TS;
    const int Mm = (m - 2) / 4 + 1;  // main-chain nodes of this sentence: ids 1, 5, ..., m-1
    // A wave holds the nodes 8 w ... 8 w + 7.  Waves without a node of the sentence only keep the barriers company, and a
    // wave's loops over its lanes' children (parents) stop at the count its first (last) node needs - both wave-uniform,
    // so that the two waves that share a SIMD when the sentence has more than 32 main-chain nodes split the work of one.
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool wave_active = 8 * wave < Mm;
    const int nr_children = wave_active ? (Mm - 8 * wave + 7) / 8 : 0;
    const int nr_parents = wave_active ? wave + 1 : 0;
    // ---- tables: everything -inf, then the emissions (base 2)
    for (int i = tid; i < 8 * Mc * TS; i += NT3) lds[i] = NEG_INF_F;
    __syncthreads();
    for (int i = tid; i < Mm * n; i += NT3) {
        const int a_id = i / n, s = i - a_id * n, a = 4 * a_id + 1;
        tb.M0[tb.at(a_id, s)] = log2_of(match[(size_t)a * T + s]);
        if (a_id > 0) {
            tb.M1[tb.at(a_id, s)] = log2_of(match[(size_t)(a - 1) * T + s]);
            tb.M3[tb.at(a_id, s)] = log2_of(match[(size_t)(a - 3) * T + s]);
        }
    }
    __syncthreads();
    const int last = Mm - 1;
    if (tid == 0) tb.S[tb.at(last, n - 1)] = tb.M0[tb.at(last, n - 1)];  // :142-147

    // ---- inside sweep: node g, right children g + l + 8 r
    {
        float A0[NR], A1[NR], A3[NR];
        const int a = 4 * g + 1;
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const int c_id = g + l + 8 * r;
            A0[r] = A1[r] = A3[r] = NEG_INF_F;
            if (g < Mm && c_id < Mm) {
                const float *row = links + (size_t)a * 4 * L + (4 * c_id + 1);
                A0[r] = log2_of(row[0]);
                if (g > 0) {  // (the root has no left option: bb runs from max(a - 3, 1) = a to a)
                    A1[r] = log2_of(row[(size_t)1 * L]);
                    A3[r] = log2_of(row[(size_t)3 * L]);
                }
            }
        }
        __syncthreads();
        // The zeros of the gradients (the rule gradients are 4 L^2 floats per sentence, of which this kernel computes the
        // main-chain entries) are issued here and drain underneath the sweeps, whose barriers wait for LDS only.
        for (int i = tid; i < L * T; i += NT3) mg[i] = 0.0f;
        {
            float4 *lg4 = reinterpret_cast<float4 *>(lg);  // (4 L^2 floats per sentence; the base is 16-byte aligned: checked by the host)
            const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int i = tid; i < L * L; i += NT3) lg4[i] = z;
        }
        float R1p = NEG_INF_F, R3p = NEG_INF_F;  // R_1, R_3 of the column one step back
        for (int t = n - 1; t >= 1; t--) {
            float R1 = NEG_INF_F, R3 = NEG_INF_F;
            if (wave_active) {
                // (children beyond the sentence have -inf rules; their table reads are clamped to a row that exists)
                float x0[NR], x1[NR], x3[NR];
                float m0 = NEG_INF_F, m1 = NEG_INF_F, m3 = NEG_INF_F;
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    if (r >= nr_children) break;
                    const int c_id = g + l + 8 * r;
                    const float x = tb.S[tb.at(c_id < Mc ? c_id : Mc - 1, t)];
                    x0[r] = A0[r] + x;
                    x1[r] = A1[r] + x;
                    x3[r] = A3[r] + x;
                    m0 = fmaxf(m0, x0[r]);
                    m1 = fmaxf(m1, x1[r]);
                    m3 = fmaxf(m3, x3[r]);
                }
                const float f0 = (m0 > NEG_INF_F) ? m0 : 0.f, f1 = (m1 > NEG_INF_F) ? m1 : 0.f, f3 = (m3 > NEG_INF_F) ? m3 : 0.f;
                float s0 = 0.f, s1 = 0.f, s3 = 0.f;
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    if (r >= nr_children) break;
                    s0 += __builtin_amdgcn_exp2f(x0[r] - f0);
                    s1 += __builtin_amdgcn_exp2f(x1[r] - f1);
                    s3 += __builtin_amdgcn_exp2f(x3[r] - f3);
                }
                const float R0 = g8_lse(m0, s0);
                R1 = g8_lse(m1, s1);
                R3 = g8_lse(m3, s3);
                const int s = t - 1;
                float term = NEG_INF_F;
                if (g < Mm) {
                    if (l == 0) {
                        tb.R0[tb.at(g, t)] = R0;
                        term = tb.M0[tb.at(g, s)] + R0;
                    } else if (l == 1) {
                        tb.R1[tb.at(g, t)] = R1;
                        term = tb.M1[tb.at(g, s)] + tb.M0[tb.at(g, s + 1)] + R1p;
                    } else if (l == 2) {
                        tb.R3[tb.at(g, t)] = R3;
                        term = tb.M3[tb.at(g, s)] + tb.M0[tb.at(g, s + 1)] + R3p;
                    }
                }
                const float val = g8_lse(term, 1.0f);
                if (g < Mm && l == 0) tb.S[tb.at(g, s)] = val;
            }
            R1p = R1;
            R3p = R3;
            lds_barrier();
        }
    }
    for (int i = tid; i < Mc * TS_out; i += NT3) {  // the table in the reference's form: natural logarithms, -inf where undefined
        const int a_id = i / TS_out, s2 = i - a_id * TS_out;
        S_out[i] = tb.S[tb.at(a_id, s2)] * LN2_F;
    }
    const float ll2 = tb.S[tb.at(0, 0)];
    if (!(ll2 > NEG_INF_F) || ll2 != ll2 || ll2 == __builtin_huge_valf()) return;  // invalid sentence: zero gradients

    // ---- outside sweep: node g, parents g - l - 8 r; V[c][t] = log2 of (outside weight / inside value)
    float At0[NR], At1[NR], At3[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const int a_id = g - l - 8 * r;
        At0[r] = At1[r] = At3[r] = NEG_INF_F;
        if (g < Mm && a_id >= 0) {
            const float *row = links + (size_t)(4 * a_id + 1) * 4 * L + (4 * g + 1);
            At0[r] = log2_of(row[0]);
            if (a_id > 0) {
                At1[r] = log2_of(row[(size_t)1 * L]);
                At3[r] = log2_of(row[(size_t)3 * L]);
            }
        }
    }
    if (tid < 2 * 3 * MC3_MAX) (&s_u[0][0][0])[tid] = NEG_INF_F;
    __syncthreads();
    if (tid == 0) {
        tb.V[tb.at(0, 0)] = -ll2;
        s_u[0][0][0] = -ll2 + tb.M0[tb.at(0, 0)];  // u_0 of the root for column 1
    }
    __syncthreads();
    for (int t = 1; t <= n - 1; t++) {
        const int buf = (t - 1) & 1;
        if (wave_active) {
            float m_ = NEG_INF_F;
            float x0[NR], x1[NR], x3[NR];
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if (r >= nr_parents) break;
                const int a_id = g - l - 8 * r, ai = a_id >= 0 ? a_id : 0;  // (no parent: -inf rules, a read that exists)
                x0[r] = At0[r] + s_u[buf][0][ai];
                x1[r] = At1[r] + s_u[buf][1][ai];
                x3[r] = At3[r] + s_u[buf][2][ai];
                m_ = fmaxf(m_, fmaxf(x0[r], fmaxf(x1[r], x3[r])));
            }
            const float f_ = (m_ > NEG_INF_F) ? m_ : 0.f;
            float s_ = 0.f;
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if (r >= nr_parents) break;
                s_ += __builtin_amdgcn_exp2f(x0[r] - f_) + __builtin_amdgcn_exp2f(x1[r] - f_) + __builtin_amdgcn_exp2f(x3[r] - f_);
            }
            const float Z = g8_lse(m_, s_);
            if (g < Mm) {
                const float v1 = tb.V[tb.at(g, t - 1)];  // (written by this node's own lane 0 one step ago)
                if (l == 0) {
                    tb.V[tb.at(g, t)] = Z;
                    s_u[buf ^ 1][0][g] = Z + tb.M0[tb.at(g, t)];
                } else if (l == 1) {
                    s_u[buf ^ 1][1][g] = v1 + tb.M1[tb.at(g, t - 1)] + tb.M0[tb.at(g, t)];
                } else if (l == 2) {
                    s_u[buf ^ 1][2][g] = v1 + tb.M3[tb.at(g, t - 1)] + tb.M0[tb.at(g, t)];
                }
            }
        }
        lds_barrier();
    }
    __syncthreads();  // (also: the zeros of the gradients have reached memory before anything is written over them)

    // ---- emission gradients from the masses of the three options of every (node, position)
    const float gw = seed_weight(grad_out, b, n, seed);
    for (int i = tid; i < Mm * n; i += NT3) {
        const int a_id = i / n, s = i - a_id * n, a = 4 * a_id + 1;
        const float v = tb.V[tb.at(a_id, s)];
        float own = __builtin_amdgcn_exp2f(v + tb.M0[tb.at(a_id, s)] + tb.R0[tb.at(a_id, s + 1)]);
        if (a_id == last && s == n - 1) own += __builtin_amdgcn_exp2f(v + tb.S[tb.at(a_id, s)]);  // :379-382
        if (a_id > 0) {
            const float m0n = tb.M0[tb.at(a_id, s + 1)];
            mg[(size_t)(a - 1) * T + s] = gw * __builtin_amdgcn_exp2f(v + tb.M1[tb.at(a_id, s)] + m0n + tb.R1[tb.at(a_id, s + 2)]);
            mg[(size_t)(a - 3) * T + s] = gw * __builtin_amdgcn_exp2f(v + tb.M3[tb.at(a_id, s)] + m0n + tb.R3[tb.at(a_id, s + 2)]);
            if (s > 0) {  // the options that started one position earlier emit this node's token here
                const float vp = tb.V[tb.at(a_id, s - 1)], m0 = tb.M0[tb.at(a_id, s)];
                own += __builtin_amdgcn_exp2f(vp + tb.M1[tb.at(a_id, s - 1)] + m0 + tb.R1[tb.at(a_id, s + 1)]);
                own += __builtin_amdgcn_exp2f(vp + tb.M3[tb.at(a_id, s - 1)] + m0 + tb.R3[tb.at(a_id, s + 1)]);
            }
        }
        mg[(size_t)a * T + s] = gw * own;
    }
    __syncthreads();
    // ---- rule gradients: U_k[a][t] = log2 of (outside weight of a starting option k that reaches column t) into the place
    // of the row sums, then one sum over the columns per (parent, option, child)
    for (int i = tid; i < Mm * n; i += NT3) {
        const int a_id = i / n, t = i - a_id * n;
        float u0 = NEG_INF_F, u1 = NEG_INF_F, u3 = NEG_INF_F;
        if (t >= 1) u0 = tb.V[tb.at(a_id, t - 1)] + tb.M0[tb.at(a_id, t - 1)];
        if (t >= 2 && a_id > 0) {
            const float w = tb.V[tb.at(a_id, t - 2)] + tb.M0[tb.at(a_id, t - 1)];
            u1 = w + tb.M1[tb.at(a_id, t - 2)];
            u3 = w + tb.M3[tb.at(a_id, t - 2)];
        }
        tb.R0[tb.at(a_id, t)] = u0;
        tb.R1[tb.at(a_id, t)] = u1;
        tb.R3[tb.at(a_id, t)] = u3;
    }
    __syncthreads();
    if (g < Mm) {
        float acc0[NR], acc1[NR], acc3[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) acc0[r] = acc1[r] = acc3[r] = 0.f;
        for (int t = 1; t <= n - 1; t++) {
            const float sc = tb.S[tb.at(g, t)];
            if (!(sc > NEG_INF_F)) continue;
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if (r >= nr_parents) break;
                const int a_id = g - l - 8 * r;
                if (a_id >= 0) {
                    acc0[r] += __builtin_amdgcn_exp2f(At0[r] + tb.R0[tb.at(a_id, t)] + sc);
                    acc1[r] += __builtin_amdgcn_exp2f(At1[r] + tb.R1[tb.at(a_id, t)] + sc);
                    acc3[r] += __builtin_amdgcn_exp2f(At3[r] + tb.R3[tb.at(a_id, t)] + sc);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const int a_id = g - l - 8 * r;
            if (a_id >= 0) {
                float *row = lg + (size_t)(4 * a_id + 1) * 4 * L + (4 * g + 1);
                row[0] = gw * acc0[r];
                row[(size_t)1 * L] = gw * acc1[r];
                row[(size_t)3 * L] = gw * acc3[r];
            }
        }
    }
}

bool g_ml3_tuned = true;

}  // namespace

bool ml3_tuned_on() { return g_ml3_tuned; }

bool inside_ml3_supported(int64_t L, int64_t T) {
    if (!g_ml3_tuned || L < 6) return false;
    const int64_t Mc = (L - 2) / 4 + 1;
    return Mc <= MC3_MAX && T <= T3_MAX;
}

int inside_ml3_forward_backward(const float *grad_output, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl,
                                float *S, float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, Seed seed,
                                void *stream) {
    const int Mc = (int)((L - 2) / 4 + 1);
    const size_t bytes = (size_t)8 * Mc * (T + 3) * sizeof(float);
#define PCFGNAT_ML3_LAUNCH(NR)                                                                                                          \
    do {                                                                                                                                \
        PCFGNAT_DYNAMIC_LDS(inside_fused_ml3_kernel<NR>, bytes);                                                                        \
        hipLaunchKernelGGL(inside_fused_ml3_kernel<NR>, dim3((unsigned)B), dim3(NT3), bytes, (hipStream_t)stream, grad_output, match_all, \
                           links, ol, tl, S, match_all_grad, links_grad, (int)L, (int)T, Mc, seed);                                      \
    } while (0)
    if (Mc <= 16) PCFGNAT_ML3_LAUNCH(2);
    else if (Mc <= 32) PCFGNAT_ML3_LAUNCH(4);
    else if (Mc <= 48) PCFGNAT_ML3_LAUNCH(6);
    else PCFGNAT_ML3_LAUNCH(8);
#undef PCFGNAT_ML3_LAUNCH
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

}  // namespace pcfgnat

extern "C" int pcfgnat_max_left3_tuned(int on) {
    const int was = pcfgnat::g_ml3_tuned ? 1 : 0;
    if (on >= 0) pcfgnat::g_ml3_tuned = on != 0;
    return was;
}

extern "C" int pcfgnat_max_left3_counts(unsigned long long *served, unsigned long long *left_to_plain, int reset) {
    unsigned long long h[2] = {0, 0};
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(h, HIP_SYMBOL(pcfgnat::g_ml3_counts), sizeof(h)));
    if (served) *served = h[0];
    if (left_to_plain) *left_to_plain = h[1];
    if (reset) {
        const unsigned long long z[2] = {0, 0};
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(pcfgnat::g_ml3_counts), z, sizeof(z)));
    }
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_max_left3_supported(int64_t L, int64_t T) { return pcfgnat::inside_ml3_supported(L, T) ? 1 : 0; }
