// General max_left ("ml" = links.size(2) - 1 = 2^left_tree_layer - 1): the inside loss, its exact backward, the best-tree
// trace and the viterbi tables for any ml other than 1 (ml = 1, the setting of every shipped script, has its own tuned
// kernels in inside.hip / viterbi.hip; at ml = 3 the loss and the viterbi tables of sentences without composite local
// trees are taken by inside_ml3.hip / viterbi.hip, and the kernels here skip them).
//
// Replaces the general-ml paths of the reference's pcfg_loss.cu (:84-349), pcfg_loss_backward.cu (:28-603),
// pcfg_best_tree.cu (:64-301) and pcfg_viterbi.cu (:22-241).
//
// Correct-but-plain design: one workgroup per sentence, the loops of the reference kept as they are with the outermost
// row loop spread over the threads and a workgroup barrier wherever the reference has a dependency between steps.
// Tables live in global memory (L2-resident).  Scatter-adds of the backward use float atomics.
#include "common.hip.h"

namespace pcfgnat {
namespace {

constexpr int NTG = 256;

struct Dims {
    int L, T, ml, Mc, Lc, TS, G;  // TS = T+2, G = ml+2
    __host__ __device__ Dims(int L_, int T_, int ml_) : L(L_), T(T_), ml(ml_) {
        Mc = (L - 2) / (ml + 1) + 1;
        Lc = L - Mc;
        TS = T + 2;
        G = ml + 2;
    }
    __device__ int mc_i2e(int x) const { return x * (ml + 1) + 1; }
    __device__ int mc_e2i(int x) const { return (x - 1) / (ml + 1); }
    __device__ int lt_i2e(int x) const { return x == 0 ? 0 : x + (x - 1) / (ml > 0 ? ml : 1) + 1; }
    __device__ int lt_e2i(int x) const { return x == 0 ? 0 : x - (x - 1) / (ml + 1) - 1; }
    __device__ int lo(int a) const { return ((a - 1) / (ml + 1)) * (ml + 1) + 1; }
    __device__ int hi(int a) const { return ((a - 1) / (ml + 1) + 1) * (ml + 1) + 1; }
    __device__ size_t s_at(int a_id, int s) const { return (size_t)a_id * TS + s; }
    __device__ size_t c_at(int b_id, int i, int g) const { return ((size_t)b_id * TS + i) * G + g; }
    __device__ size_t lk(int a, int k, int c) const { return ((size_t)a * (ml + 1) + k) * L + c; }
    __host__ __device__ size_t s_size() const { return (size_t)Mc * TS; }
    __host__ __device__ size_t c_size() const { return (size_t)Lc * TS * G; }
    // aux per sentence: C | Cg | Ct (c_size each) | Sg | St (s_size each); Ct/St are the best-tree marks
    __host__ __device__ size_t aux_floats() const { return 3 * c_size() + 2 * s_size(); }
};

// The kernels are templates over the table type RT (float, or double: the reference dispatches both, pcfg_loss.cu:395).
template <typename RT>
__device__ __forceinline__ RT neg_inf();
template <>
__device__ __forceinline__ float neg_inf<float>() { return NEG_INF_F; }
template <>
__device__ __forceinline__ double neg_inf<double>() { return -__builtin_huge_val(); }
__device__ __forceinline__ float rexp(float x) { return expf(x); }
__device__ __forceinline__ double rexp(double x) { return exp(x); }
__device__ __forceinline__ float rlog(float x) { return logf(x); }
__device__ __forceinline__ double rlog(double x) { return log(x); }
__device__ __forceinline__ float rmax(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double rmax(double a, double b) { return fmax(a, b); }
__device__ __forceinline__ bool is_inf(float x) { return fabsf(x) == __builtin_huge_valf(); }
__device__ __forceinline__ bool is_inf(double x) { return fabs(x) == __builtin_huge_val(); }
template <typename RT>
__device__ __forceinline__ bool bad(RT v) { return v != v; }
// Cells that other threads update with (L2) atomics must not be read through a possibly stale L1 line.
template <typename RT>
__device__ __forceinline__ RT coherent_load(const RT *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool len_ok(const Dims &d, int m, int n) {
    return m >= d.ml + 3 && m <= d.L && ((m - 2) % (d.ml + 1)) == 0 && n >= 2 && n <= d.T;
}

// Sentences that the one-launch kernel for max_left = 3 (inside_ml3.hip) has served: everything except valid sentences
// that hold a rule of a composite local tree.  Only asked when that kernel ran in front (skip_ml3_taken).
__device__ __forceinline__ bool taken_by_ml3(int skip_ml3_taken, const float *links, const Dims &d, int m, int n, int tid) {
    if (!skip_ml3_taken) return false;  // (uniform)
    if (!len_ok(d, m, n)) return true;
    return !ml3_composite_rules<NTG>(links, d.L, m, tid);
}
__device__ __forceinline__ bool taken_by_ml3(int, const double *, const Dims &, int, int, int) { return false; }
// The same for the Viterbi tables (viterbi_ml3_kernel): a sentence of valid size is left over only if it holds such a rule.
__device__ __forceinline__ bool viterbi_taken_by_ml3(int skip_ml3_taken, const float *links, int L, int m, int tid) {
    if (!skip_ml3_taken) return false;  // (uniform)
    if (m < 2 || m > L || ((m - 2) % 4) != 0) return true;
    return !ml3_composite_rules<NTG>(links, L, m, tid);
}
__device__ __forceinline__ bool viterbi_taken_by_ml3(int, const double *, int, int, int) { return false; }

// ---- inside forward (pcfg_loss.cu:262-349 then :84-224) -----------------------------------------------------
template <typename RT>
__global__ __launch_bounds__(NTG) void generic_fwd_kernel(const RT *__restrict__ match_all, const RT *__restrict__ links_all,
                                                         const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                         RT *__restrict__ S_all, RT *__restrict__ aux_all, int L, int T, int ml,
                                                         int skip_ml3_taken) {
    const Dims d(L, T, ml);
    const int b = blockIdx.x, tid = threadIdx.x;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const RT *match = match_all + (size_t)b * L * T;
    const RT *links = links_all + (size_t)b * L * (ml + 1) * L;
    if (taken_by_ml3(skip_ml3_taken, links, d, m, n, tid)) return;
    RT *S = S_all + (size_t)b * d.s_size();
    RT *C = aux_all + (size_t)b * d.aux_floats();
    for (size_t i = tid; i < d.s_size(); i += NTG) S[i] = neg_inf<RT>();
    if (!len_ok(d, m, n)) {
        __syncthreads();
        if (tid == 0) S[0] = (RT)__builtin_nanf("");
        return;
    }
    for (size_t i = tid; i < d.c_size(); i += NTG) C[i] = neg_inf<RT>();
    __syncthreads();
    // :288-300
    for (int i = tid; i <= n; i += NTG) C[d.c_at(0, i, 0)] = 0.f;
    for (int w = tid; w < d.Lc * n; w += NTG) {
        const int a_id = w / n, i = w - a_id * n;
        const int a = d.lt_i2e(a_id);
        if (a > 0 && a < m && ((a - d.lo(a)) % 2 == 1)) C[d.c_at(a_id, i, 1)] = match[(size_t)a * T + i];
    }
    __syncthreads();
    // :301-348
    for (int gap = 2; gap < ml + 2; gap++) {
        const int ni = n - gap - 1;
        for (int w = tid; ni > 0 && w < d.Lc * ni; w += NTG) {
            const int a_id = w / ni, i = w - a_id * ni;
            const int a = d.lt_i2e(a_id);
            if (!(a > 0 && a < m)) continue;
            const int hi = d.hi(a), b_start = a - ml < 1 ? 1 : a - ml;
            RT maxval = neg_inf<RT>();
            for (int pass = 0; pass < 2; pass++) {
                RT sum = 0.f;
                for (int j = 0; j < gap; j++)
                    for (int bb = b_start; bb < a + 1; bb++) {
                        const int b_id = d.lt_e2i(bb == a ? 0 : bb);
                        for (int c = a + 1; c < hi && c < m; c++) {
                            RT t = links[d.lk(a, a - bb, c)] + C[d.c_at(b_id, i, j)] + C[d.c_at(d.lt_e2i(c), i + j + 1, gap - j - 1)] +
                                      match[(size_t)a * T + i + j];
                            if (bad(t)) t = neg_inf<RT>();
                            if (pass == 0) maxval = rmax(maxval, t);
                            else sum += rexp(t - maxval);
                        }
                    }
                if (pass == 0 && maxval == neg_inf<RT>()) break;
                if (pass == 1) C[d.c_at(a_id, i, gap)] = rlog(sum) + maxval;
            }
        }
        __syncthreads();
    }
    // :142-147
    if (tid == 0) S[d.s_at(d.mc_e2i(m - 1), n - 1)] = match[(size_t)(m - 1) * T + (n - 1)];
    __syncthreads();
    // :148-214
    for (int start = n - 2; start >= 0; start--) {
        for (int a_id = tid; a_id < d.Mc; a_id += NTG) {
            const int a = d.mc_i2e(a_id);
            if (!(a > 0 && a < m)) continue;
            const int b_start = a - ml < 1 ? 1 : a - ml;
            RT maxval = neg_inf<RT>();
            for (int pass = 0; pass < 2; pass++) {
                RT sum = 0.f;
                for (int c_id = a_id; d.mc_i2e(c_id) < m; c_id++) {
                    const int c = d.mc_i2e(c_id);
                    for (int j = 0; j < n - start && j < ml + 1; j++)
                        for (int bb = b_start; bb < a + 1; bb++) {
                            const int b_id = d.lt_e2i(bb == a ? 0 : bb);
                            RT t = links[d.lk(a, a - bb, c)] + S[d.s_at(c_id, start + j + 1)] + C[d.c_at(b_id, start, j)] +
                                      match[(size_t)a * T + start + j];
                            if (bad(t)) t = neg_inf<RT>();
                            if (pass == 0) maxval = rmax(maxval, t);
                            else sum += rexp(t - maxval);
                        }
                }
                if (pass == 0 && maxval == neg_inf<RT>()) break;
                if (pass == 1) S[d.s_at(a_id, start)] = rlog(sum) + maxval;
            }
        }
        __syncthreads();
    }
}

// ---- backward: exact gradient of the recurrences above (organised like pcfg_loss_backward.cu:28-603) ------------
template <typename RT>
__global__ __launch_bounds__(NTG) void generic_bwd_kernel(const RT *__restrict__ grad_out, const RT *__restrict__ S_all,
                                                         RT *__restrict__ aux_all, const RT *__restrict__ match_all,
                                                         const RT *__restrict__ links_all, const int64_t *__restrict__ out_len,
                                                         const int64_t *__restrict__ tgt_len, RT *__restrict__ mg_all,
                                                         RT *__restrict__ lg_all, int L, int T, int ml, Seed seed, int skip_ml3_taken) {
    const Dims d(L, T, ml);
    const int b = blockIdx.x, tid = threadIdx.x;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const RT *match = match_all + (size_t)b * L * T;
    const RT *links = links_all + (size_t)b * L * (ml + 1) * L;
    if (taken_by_ml3(skip_ml3_taken, links, d, m, n, tid)) return;
    const RT *S = S_all + (size_t)b * d.s_size();
    RT *aux = aux_all + (size_t)b * d.aux_floats();
    const RT *C = aux;
    RT *Cg = aux + d.c_size();
    RT *Sg = aux + 3 * d.c_size();
    RT *mg = mg_all + (size_t)b * L * T;
    RT *lg = lg_all + (size_t)b * L * (ml + 1) * L;
    for (size_t i = tid; i < (size_t)L * T; i += NTG) mg[i] = 0.f;
    for (size_t i = tid; i < (size_t)L * (ml + 1) * L; i += NTG) lg[i] = 0.f;
    const RT ll = S[0];
    if (!len_ok(d, m, n) || ll != ll || is_inf(ll)) return;  // invalid sentence: zero gradients
    for (size_t i = tid; i < d.s_size(); i += NTG) Sg[i] = 0.f;
    for (size_t i = tid; i < d.c_size(); i += NTG) Cg[i] = 0.f;
    __syncthreads();
    const RT g = seed_weight(grad_out, b, n, seed);
    if (tid == 0) Sg[0] = g;  // :76-80
    __syncthreads();
    // main chain, start ascending (:83-112, 175-205, 348-376, 512-531)
    for (int s = 0; s < n; s++) {
        for (int a_id = tid; a_id < d.Mc; a_id += NTG) {
            const int a = d.mc_i2e(a_id);
            if (!(a > 0 && a < m)) continue;
            const RT sg = coherent_load(&Sg[d.s_at(a_id, s)]), sa = S[d.s_at(a_id, s)];
            if (sg == 0.f || sa != sa || is_inf(sa)) continue;
            const int b_start = a - ml < 1 ? 1 : a - ml;
            for (int c_id = a_id; d.mc_i2e(c_id) < m; c_id++) {
                const int c = d.mc_i2e(c_id);
                for (int j = 0; j < n - s && j < ml + 1; j++) {
                    const RT sc = S[d.s_at(c_id, s + j + 1)];
                    if (sc != sc || is_inf(sc)) continue;
                    for (int bb = b_start; bb < a + 1; bb++) {
                        const int b_id = d.lt_e2i(bb == a ? 0 : bb);
                        const RT t = links[d.lk(a, a - bb, c)] + sc + C[d.c_at(b_id, s, j)] + match[(size_t)a * T + s + j] - sa;
                        if (bad(t) || t == neg_inf<RT>()) continue;
                        const RT p = sg * rexp(t);
                        atomicAdd(&Sg[d.s_at(c_id, s + j + 1)], p);
                        if (b_id != 0) atomicAdd(&Cg[d.c_at(b_id, s, j)], p);
                        atomicAdd(&mg[(size_t)a * T + s + j], p);
                        atomicAdd(&lg[d.lk(a, a - bb, c)], p);
                    }
                }
            }
        }
        __syncthreads();
    }
    if (tid == 0) atomicAdd(&mg[(size_t)(m - 1) * T + (n - 1)], coherent_load(&Sg[d.s_at(d.mc_e2i(m - 1), n - 1)]));  // :379-382
    __syncthreads();
    // local trees, gap descending (:236-276, 407-428, 556-599; every gap >= 2, the forward's own ranges)
    for (int gap = ml + 1; gap >= 2; gap--) {
        const int ni = n - gap - 1;
        for (int w = tid; ni > 0 && w < d.Lc * ni; w += NTG) {
            const int a_id = w / ni, i = w - a_id * ni;
            const int a = d.lt_i2e(a_id);
            if (!(a > 0 && a < m)) continue;
            const RT cg = coherent_load(&Cg[d.c_at(a_id, i, gap)]), ca = C[d.c_at(a_id, i, gap)];
            if (cg == 0.f || ca != ca || is_inf(ca)) continue;
            const int hi = d.hi(a), b_start = a - ml < 1 ? 1 : a - ml;
            for (int j = 0; j < gap; j++)
                for (int bb = b_start; bb < a + 1; bb++) {
                    const int b_id = d.lt_e2i(bb == a ? 0 : bb);
                    for (int c = a + 1; c < hi && c < m; c++) {
                        const int c_id = d.lt_e2i(c);
                        const RT t = links[d.lk(a, a - bb, c)] + C[d.c_at(b_id, i, j)] + C[d.c_at(c_id, i + j + 1, gap - j - 1)] +
                                        match[(size_t)a * T + i + j] - ca;
                        if (bad(t) || t == neg_inf<RT>()) continue;
                        const RT p = cg * rexp(t);
                        if (b_id != 0) atomicAdd(&Cg[d.c_at(b_id, i, j)], p);
                        atomicAdd(&Cg[d.c_at(c_id, i + j + 1, gap - j - 1)], p);
                        atomicAdd(&mg[(size_t)a * T + i + j], p);
                        atomicAdd(&lg[d.lk(a, a - bb, c)], p);
                    }
                }
        }
        __syncthreads();
    }
    // leaves (:429-433)
    for (int w = tid; w < d.Lc * n; w += NTG) {
        const int a_id = w / n, i = w - a_id * n;
        const int a = d.lt_i2e(a_id);
        if (a > 0 && a < m && ((a - d.lo(a)) % 2 == 1)) atomicAdd(&mg[(size_t)a * T + i], coherent_load(&Cg[d.c_at(a_id, i, 1)]));
    }
}

// ---- best tree (pcfg_best_tree.cu:64-197, 239-301); the 4-lane scan order is emulated per node -----------------
template <typename RT>
__global__ __launch_bounds__(NTG) void generic_best_tree_kernel(const RT *__restrict__ S_all, RT *__restrict__ aux_all,
                                                               const RT *__restrict__ match_all, const RT *__restrict__ links_all,
                                                               const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
                                                               int64_t *__restrict__ tree_all, int L, int T, int ml) {
    const Dims d(L, T, ml);
    const int b = blockIdx.x, tid = threadIdx.x;
    const int m = (int)out_len[b], n = (int)tgt_len[b];
    const RT *match = match_all + (size_t)b * L * T;
    const RT *links = links_all + (size_t)b * L * (ml + 1) * L;
    const RT *S = S_all + (size_t)b * d.s_size();
    RT *aux = aux_all + (size_t)b * d.aux_floats();
    const RT *C = aux;
    RT *St = aux + 3 * d.c_size() + d.s_size();  // marks (0 / 1)
    RT *Ct = aux + 2 * d.c_size();
    int64_t *tree = tree_all + (size_t)b * L;
    for (int i = tid; i < L; i += NTG) tree[i] = -1;
    if (!len_ok(d, m, n)) return;
    for (size_t i = tid; i < d.s_size(); i += NTG) St[i] = 0.f;
    for (size_t i = tid; i < d.c_size(); i += NTG) Ct[i] = 0.f;
    __syncthreads();
    if (tid == 0) St[0] = 1.f;
    __syncthreads();
    for (int s = 0; s <= n; s++) {
        for (int a_id = tid; a_id < d.Mc; a_id += NTG) {
            const int a = d.mc_i2e(a_id);
            if (!(a > 0 && a < m && St[d.s_at(a_id, s)] != 0.f)) continue;
            const int b_start = a - ml < 1 ? 1 : a - ml;
            RT lane_val[4];
            int lane_c[4], lane_j[4], lane_b[4];
            for (int x = 0; x < 4; x++) {
                RT maxval = neg_inf<RT>();
                int max_c = -1, max_j = 0, max_b = -1;
                for (int c_id = a_id + x + 1; d.mc_i2e(c_id) < m; c_id += 4) {
                    const int c = d.mc_i2e(c_id);
                    for (int j = 0; j < n - s && j < ml + 1; j++)
                        for (int bb = b_start; bb < a + 1; bb++) {
                            const int b_id = d.lt_e2i(bb == a ? 0 : bb);
                            RT t = links[d.lk(a, a - bb, c)] + S[d.s_at(c_id, s + j + 1)] + C[d.c_at(b_id, s, j)] +
                                      match[(size_t)a * T + s + j];
                            if (bad(t)) t = neg_inf<RT>();
                            if (t > maxval) { maxval = t; max_c = c_id; max_j = j; max_b = b_id; }
                        }
                }
                lane_val[x] = maxval; lane_c[x] = max_c; lane_j[x] = max_j; lane_b[x] = max_b;
            }
            for (int x = 0; x < 2; x++)
                if (lane_val[x + 2] > lane_val[x]) { lane_val[x] = lane_val[x + 2]; lane_c[x] = lane_c[x + 2]; lane_j[x] = lane_j[x + 2]; lane_b[x] = lane_b[x + 2]; }
            if (lane_val[1] > lane_val[0]) { lane_val[0] = lane_val[1]; lane_c[0] = lane_c[1]; lane_j[0] = lane_j[1]; lane_b[0] = lane_b[1]; }
            if (lane_c[0] != -1 && lane_b[0] != -1) {
                St[d.s_at(lane_c[0], s + lane_j[0] + 1)] = 1.f;
                Ct[d.c_at(lane_b[0], s, lane_j[0])] = 1.f;
            }
            tree[a] = s + lane_j[0];
        }
        __syncthreads();
    }
    if (ml == 0) return;
    for (int gap = ml + 1; gap >= 1; gap--) {
        const int ni = n - gap - 1;
        for (int w = tid; ni > 0 && w < (d.Lc - 1) * ni; w += NTG) {
            const int a_id = 1 + w / ni, i = w % ni;
            const int a = d.lt_i2e(a_id);
            if (!(a > 0 && a < m) || Ct[d.c_at(a_id, i, gap)] == 0.f) continue;
            const int hi = d.hi(a), b_start = a - ml < 1 ? 1 : a - ml;
            int max_j = 0, max_b = -1, max_c = -1;
            RT maxval = neg_inf<RT>();
            for (int j = 0; j < gap; j++)
                for (int bb = b_start; bb < a + 1; bb++) {
                    const int b_id = d.lt_e2i(bb == a ? 0 : bb);
                    for (int c = a + 1; c < hi && c < m; c++) {
                        const int c_id = d.lt_e2i(c);
                        RT t = links[d.lk(a, a - bb, c)] + C[d.c_at(b_id, i, j)] + C[d.c_at(c_id, i + j + 1, gap - j - 1)] +
                                  match[(size_t)a * T + i + j];
                        if (bad(t)) t = neg_inf<RT>();
                        if (t > maxval) { maxval = t; max_j = j; max_b = b_id; max_c = c_id; }
                    }
                }
            if (max_b != -1 && max_c != -1) {
                Ct[d.c_at(max_b, i, max_j)] = 1.f;
                Ct[d.c_at(max_c, i + max_j + 1, gap - max_j - 1)] = 1.f;
            }
            tree[a] = i + max_j;
        }
        __syncthreads();
    }
}

// ---- viterbi (pcfg_viterbi.cu:177-241 then :22-140); tables [L][Lq] by external node id --------------------------
template <typename RT>
__global__ __launch_bounds__(NTG) void generic_viterbi_kernel(const RT *__restrict__ ob_all, const RT *__restrict__ links_all,
                                                             const int64_t *__restrict__ out_len, RT *__restrict__ S_all,
                                                             int64_t *__restrict__ R_all,
                                                             int64_t *__restrict__ Lt_all, int64_t *__restrict__ M_all, int L, int ml,
                                                             int skip_ml3_taken) {
    const int Lq = L / 4;
    const int b = blockIdx.x, tid = threadIdx.x;
    const int m = (int)out_len[b];
    const RT *ob = ob_all + (size_t)b * L;
    const RT *links = links_all + (size_t)b * L * (ml + 1) * L;
    if (viterbi_taken_by_ml3(skip_ml3_taken, links, L, m, tid)) return;
    const size_t tab = (size_t)b * L * Lq;
    // the local-tree table lives in the rows of S that belong to local nodes and node 0 (the S sweep only touches
    // main-chain rows); those cells are put back to -inf at the end, as the reference returns them
    RT *S = S_all + tab, *Cv = S;
    int64_t *R = R_all + tab, *Lt = Lt_all + tab, *M = M_all + tab;
    auto at = [&](int a, int l) -> size_t { return (size_t)a * Lq + l; };
    auto lk = [&](int a, int k, int c) -> size_t { return ((size_t)a * (ml + 1) + k) * L + c; };
    for (size_t i = tid; i < (size_t)L * Lq; i += NTG) { S[i] = neg_inf<RT>(); R[i] = 0; Lt[i] = 0; M[i] = 0; }
    if (m < 2 || m > L || ((m - 2) % (ml + 1)) != 0) return;
    __syncthreads();
    for (int a = 1 + tid; a < L; a += NTG) {
        const int lo = ((a - 1) / (ml + 1)) * (ml + 1) + 1;
        if (a < m && ((a - lo) % 2 == 1) && Lq > 1) Cv[at(a, 1)] = ob[a];
    }
    if (tid == 0) Cv[at(0, 0)] = 0.f;
    __syncthreads();
    for (int gap = 2; gap < ml + 1 && gap < Lq; gap++) {
        for (int a = 1 + tid; a < L; a += NTG) {
            if (!(a < m && (a % (ml + 1) != 1))) continue;
            const int hi = ((a - 1) / (ml + 1) + 1) * (ml + 1) + 1, b_start = a - ml < 1 ? 1 : a - ml;
            RT maxval = neg_inf<RT>();
            int max_b = 0, max_c = 0, max_j = 0;
            for (int j = 0; j < gap; j++)
                for (int bb = b_start; bb < a + 1; bb++) {
                    const int _b = bb == a ? 0 : bb;
                    for (int c = a + 1; c < hi && c < m; c++) {
                        RT t = ((links[lk(a, a - bb, c)] + Cv[at(_b, j)]) + Cv[at(c, gap - j - 1)]) + ob[a];
                        if (bad(t)) t = neg_inf<RT>();
                        if (t > maxval) { maxval = t; max_b = _b; max_c = c; max_j = j; }
                    }
                }
            if (maxval != neg_inf<RT>()) { Cv[at(a, gap)] = maxval; R[at(a, gap)] = max_c; Lt[at(a, gap)] = max_b; M[at(a, gap)] = max_j; }
        }
        __syncthreads();
    }
    if (tid == 0 && Lq > 1) S[at(m - 1, 1)] = ob[m - 1];
    __syncthreads();
    for (int len = 2; len < m / 4; len++) {
        for (int id = tid; id * (ml + 1) + 1 < m; id += NTG) {
            const int a = id * (ml + 1) + 1, b_start = a - ml < 1 ? 1 : a - ml;
            RT lane_val[4];
            int lane_c[4], lane_j[4], lane_b[4];
            for (int x = 0; x < 4; x++) {
                RT maxval = neg_inf<RT>();
                int max_b = 0, max_c = 0, max_j = 0;
                for (int c_id = id + x; c_id * (ml + 1) + 1 < m; c_id += 4) {
                    const int c = c_id * (ml + 1) + 1;
                    for (int j = 0; j < ml + 1; j++)
                        for (int bb = b_start; bb < a + 1; bb++) {
                            const int _b = bb == a ? 0 : bb;
                            const RT sc = (len - j - 1 >= 0) ? S[at(c, len - j - 1)] : neg_inf<RT>();
                            const RT cj = (j < Lq) ? Cv[at(_b, j)] : neg_inf<RT>();
                            RT t = ((links[lk(a, a - bb, c)] + cj) + sc) + ob[a];
                            if (bad(t)) t = neg_inf<RT>();
                            if (t > maxval) { maxval = t; max_b = _b; max_c = c; max_j = j; }
                        }
                }
                lane_val[x] = maxval; lane_c[x] = max_c; lane_j[x] = max_j; lane_b[x] = max_b;
            }
            for (int x = 0; x < 2; x++)
                if (lane_val[x + 2] > lane_val[x]) { lane_val[x] = lane_val[x + 2]; lane_c[x] = lane_c[x + 2]; lane_j[x] = lane_j[x + 2]; lane_b[x] = lane_b[x + 2]; }
            if (lane_val[1] > lane_val[0]) { lane_val[0] = lane_val[1]; lane_c[0] = lane_c[1]; lane_j[0] = lane_j[1]; lane_b[0] = lane_b[1]; }
            if (lane_val[0] != neg_inf<RT>()) {
                S[at(a, len)] = lane_val[0]; Lt[at(a, len)] = lane_b[0]; R[at(a, len)] = lane_c[0]; M[at(a, len)] = lane_j[0];
            }
        }
        __syncthreads();
    }
    for (int w = tid; w < L * Lq; w += NTG) {
        const int a = w / Lq;
        if (a == 0 || (a % (ml + 1)) != 1 || ml == 0) {
            if (a == 0 || ml > 0) S[w] = neg_inf<RT>();
        }
    }
}

}  // namespace

size_t generic_aux_floats(int64_t B, int64_t L, int64_t T, int64_t ml) { return (size_t)B * Dims((int)L, (int)T, (int)ml).aux_floats(); }

namespace {
template <typename RT>
int forward_t(const RT *match_all, const RT *links, const int64_t *ol, const int64_t *tl, RT *S, RT *aux, int64_t B, int64_t L, int64_t T,
              int64_t ml, void *stream, int skip_ml3_taken = 0) {
    hipLaunchKernelGGL(generic_fwd_kernel<RT>, dim3((unsigned)B), dim3(NTG), 0, (hipStream_t)stream, match_all, links, ol, tl, S, aux, (int)L,
                       (int)T, (int)ml, skip_ml3_taken);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
template <typename RT>
int backward_t(const RT *go, const RT *S, RT *aux, const RT *match_all, const RT *links, const int64_t *ol, const int64_t *tl, RT *mg, RT *lg,
               int64_t B, int64_t L, int64_t T, int64_t ml, Seed seed, void *stream, int skip_ml3_taken = 0) {
    hipLaunchKernelGGL(generic_bwd_kernel<RT>, dim3((unsigned)B), dim3(NTG), 0, (hipStream_t)stream, go, S, aux, match_all, links, ol, tl, mg,
                       lg, (int)L, (int)T, (int)ml, seed, skip_ml3_taken);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
template <typename RT>
int best_tree_t(const RT *S, RT *aux, const RT *match_all, const RT *links, const int64_t *ol, const int64_t *tl, int64_t *tree, int64_t B,
                int64_t L, int64_t T, int64_t ml, void *stream) {
    hipLaunchKernelGGL(generic_best_tree_kernel<RT>, dim3((unsigned)B), dim3(NTG), 0, (hipStream_t)stream, S, aux, match_all, links, ol, tl,
                       tree, (int)L, (int)T, (int)ml);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
template <typename RT>
int viterbi_t(const RT *ob, const RT *links, const int64_t *ol, RT *S, int64_t *R, int64_t *Lt, int64_t *M, int64_t B, int64_t L, int64_t ml,
              void *stream, int skip_ml3_taken = 0) {
    hipLaunchKernelGGL(generic_viterbi_kernel<RT>, dim3((unsigned)B), dim3(NTG), 0, (hipStream_t)stream, ob, links, ol, S, R, Lt, M, (int)L,
                       (int)ml, skip_ml3_taken);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

int check_f64(const char *who, int64_t B, int64_t L, int64_t T, int64_t ml) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 4 && T >= 2, "%s: need B >= 0, L >= 4, T >= 2 (got B=%lld L=%lld T=%lld)", who, (long long)B,
                    (long long)L, (long long)T);
    PCFGNAT_REQUIRE(L <= 4096 && T <= 4096 && B <= 65535, "%s: dimension too large (L, T <= 4096, B <= 65535)", who);
    PCFGNAT_REQUIRE(ml >= 0 && ml <= 63 && L >= ml + 3, "%s: max_left = %lld needs a graph of at least max_left + 3 nodes (and max_left <= 63)",
                    who, (long long)ml);
    return PCFGNAT_OK;
}
}  // namespace

int generic_forward(const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux, int64_t B,
                    int64_t L, int64_t T, int64_t ml, void *stream, int skip_ml3_taken) {
    return forward_t<float>(match_all, links, ol, tl, S, aux, B, L, T, ml, stream, skip_ml3_taken);
}

int generic_backward(const float *go, const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol,
                     const int64_t *tl, float *mg, float *lg, int64_t B, int64_t L, int64_t T, int64_t ml, Seed seed, void *stream,
                     int skip_ml3_taken) {
    return backward_t<float>(go, S, aux, match_all, links, ol, tl, mg, lg, B, L, T, ml, seed, stream, skip_ml3_taken);
}

int generic_best_tree(const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl,
                      int64_t *tree, int64_t B, int64_t L, int64_t T, int64_t ml, void *stream) {
    return best_tree_t<float>(S, aux, match_all, links, ol, tl, tree, B, L, T, ml, stream);
}

int generic_viterbi(const float *ob, const float *links, const int64_t *ol, float *S, int64_t *R, int64_t *Lt, int64_t *M, int64_t B,
                    int64_t L, int64_t ml, void *stream, int skip_ml3_taken) {
    return viterbi_t<float>(ob, links, ol, S, R, Lt, M, B, L, ml, stream, skip_ml3_taken);
}

}  // namespace pcfgnat

using namespace pcfgnat;

// ---- float64 entry points: every max_left (1 included) runs the plain kernels above ---------------------------------
extern "C" size_t pcfgnat_pcfg_aux_elems_f64(int64_t B, int64_t L, int64_t T, int64_t ml) {
    if (B <= 0 || L < 4 || T < 2 || ml < 0 || L < ml + 3) return 0;
    return generic_aux_floats(B, L, T, ml);
}

extern "C" int pcfgnat_pcfg_loss_f64(const double *match_all, const double *links, const int64_t *output_length,
                                     const int64_t *target_length, double *S, double *aux, int64_t B, int64_t L, int64_t T, int64_t ml,
                                     void *stream) {
    int rc = check_f64("pcfg_loss_f64", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(match_all && links && output_length && target_length && S && aux, "pcfg_loss_f64: null pointer");
    return forward_t<double>(match_all, links, output_length, target_length, S, aux, B, L, T, ml, stream);
}

extern "C" int pcfgnat_pcfg_loss_backward_f64(const double *grad_output, const double *S, double *aux, const double *match_all,
                                              const double *links, const int64_t *output_length, const int64_t *target_length,
                                              double *match_all_grad, double *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                              void *stream) {
    int rc = check_f64("pcfg_loss_backward_f64", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(grad_output && S && aux && match_all && links && output_length && target_length && match_all_grad && links_grad,
                    "pcfg_loss_backward_f64: null pointer");
    return backward_t<double>(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T, ml,
                              seed_of(B), stream);
}

extern "C" int pcfgnat_pcfg_best_tree_f64(const double *S, double *aux, const double *match_all, const double *links,
                                          const int64_t *output_length, const int64_t *target_length, int64_t *tree, int64_t B, int64_t L,
                                          int64_t T, int64_t ml, void *stream) {
    int rc = check_f64("pcfg_best_tree_f64", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(S && aux && match_all && links && output_length && target_length && tree, "pcfg_best_tree_f64: null pointer");
    return best_tree_t<double>(S, aux, match_all, links, output_length, target_length, tree, B, L, T, ml, stream);
}

extern "C" int pcfgnat_pcfg_viterbi_f64(const double *ob_lprob, const double *links, const int64_t *output_length, double *S, int64_t *R,
                                        int64_t *Lt, int64_t *M, int64_t B, int64_t L, int64_t ml, void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 4 && L <= 4096, "pcfg_viterbi_f64: need B >= 0 and 4 <= L <= 4096 (got B=%lld L=%lld)", (long long)B,
                    (long long)L);
    PCFGNAT_REQUIRE(ml >= 0 && ml <= 63 && L / 4 > ml, "pcfg_viterbi_f64: max_left out of range for this graph size");
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(ob_lprob && links && output_length && S && R && Lt && M, "pcfg_viterbi_f64: null pointer");
    return viterbi_t<double>(ob_lprob, links, output_length, S, R, Lt, M, B, L, ml, stream);
}
