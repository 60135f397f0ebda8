// GLAT best-tree trace over the inside tables (max_left = 1), alone and followed by the criterion's glancing glue.
// Part of inside.hip (one translation unit: the kernels share helpers and the anonymous namespace).
#pragma once
#include "inside_common.hip.h"

namespace pcfgnat {
namespace {

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

}  // namespace
}  // namespace pcfgnat
