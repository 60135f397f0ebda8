/*
 * TEST INFRASTRUCTURE ONLY - CPU restatement of the PCFG-NAT structured-loss path.
 *
 * This body is included twice by pcfg_oracle.c, once with REAL=float (suffix _f32) and once with
 * REAL=double (suffix _f64).  Only tests, the smoke check and the cpu_baseline leg of the benchmark
 * may call it; the product path never does.
 *
 * Every function follows the loops of the reference kernel it cites (paths are relative to the
 * reference's fs_plugins/custom_ops/), one sentence at a time, sequentially inside a sentence and
 * (optionally) OpenMP-parallel over the batch.  General max_left ("ml") is supported.
 *
 * Deliberate deviations from the reference (all vanish on inputs the model can produce):
 *   - the backward is the exact gradient of the forward recurrences: the S_grad scatter includes the
 *     self child c == a (reference: a < c only, pcfg_loss_backward.cu:87) and the local-tree part
 *     handles every gap >= 2 with the forward's own child ranges (reference: gap > 2 only, an
 *     EPSILON cut and narrower ranges, pcfg_loss_backward.cu:236-276, 407, 556-568);
 *   - "float res" (pcfg_loss.cu:182, 319) truncates the fp64 tables of the reference to fp32; the
 *     _f64 variant here keeps full double precision;
 *   - the viterbi read S[c][len-j-1] with len-j-1 < 0 (pcfg_viterbi.cu:83, only for ml >= 2) is
 *     treated as -inf instead of reading out of bounds.
 *
 * Parity pins (see tests/test_oracle_*.py): brute-force enumeration of derivations on tiny graphs
 * (inside log-likelihood, viterbi scores and yields, best-tree choices), central finite differences
 * and the token/rule mass invariants (gradients), torch.log_softmax/gather (logsoftmax_gather).
 */

#define MC_I2E(x) ((x) * (ml + 1) + 1)
#define MC_E2I(x) (((x) - 1) / (ml + 1))
#define LT_I2E(x) (((x) == 0) ? 0 : ((x) + ((x) - 1) / ml + 1))
#define LT_E2I(x) (((x) == 0) ? 0 : ((x) - ((x) - 1) / (ml + 1) - 1))

#define S_AT(t, a_id, s) (t)[(size_t)(a_id) * (T + 2) + (s)]
#define C_AT(t, b_id, i, g) (t)[((size_t)(b_id) * (T + 2) + (i)) * (ml + 2) + (g)]
#define LK(a, k, c) links[((size_t)(a) * (ml + 1) + (k)) * L + (c)]
#define MA(a, i) match[(size_t)(a) * T + (i)]

#define NEG_INF (-(REAL)INFINITY)

/* ---------------------------------------------------------------------------------------------
 * logsoftmax_gather  (logsoftmax_gather.cu:238-292)
 * x: [rows, V] (already widened to REAL), idx: [rows, T] int64 with element strides
 * (idx_row_stride, idx_col_stride) after the caller has folded the batch/position strides into a
 * per-row base offset table `idx_base[rows]`.  sel: [rows, T].  If probs != NULL the softmax of the
 * row is written there (the reference writes it over the logits, :278-289).
 * ------------------------------------------------------------------------------------------- */
void FN(oracle_lsg_fwd)(const REAL *x, const int64_t *idx, const int64_t *idx_base, int64_t idx_col_stride,
                        REAL *sel, REAL *probs, int64_t rows, int64_t V, int64_t T)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const REAL *xr = x + r * V;
        REAL mx = NEG_INF;
        for (int64_t v = 0; v < V; v++)
            if (xr[v] > mx) mx = xr[v]; /* :251-260 */
        REAL sum = 0;
        for (int64_t v = 0; v < V; v++) sum += EXP(xr[v] - mx); /* :261-270 */
        REAL lg = LOG(sum);
        for (int64_t s = 0; s < T; s++) { /* :273-276 */
            int64_t t = idx[idx_base[r] + s * idx_col_stride];
            sel[r * T + s] = (xr[t] - mx) - lg;
        }
        if (probs) {
            REAL *pr = probs + r * V;
            for (int64_t v = 0; v < V; v++) pr[v] = EXP(xr[v] - mx) / sum; /* :285 */
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Backward of logsoftmax_gather as the autograd wrapper performs it (pcfg_loss.py:176-177), in REAL
 * arithmetic: buf = probs * -(sum_s g[s]); buf[idx[s]] += g[s] for s ascending.  In place on `buf`.
 * ------------------------------------------------------------------------------------------- */
void FN(oracle_lsg_bwd)(REAL *buf, const int64_t *idx, const int64_t *idx_base, int64_t idx_col_stride, const REAL *g,
                        int64_t rows, int64_t V, int64_t T)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        REAL *br = buf + r * V;
        REAL sum = 0;
        for (int64_t s = 0; s < T; s++) sum += g[r * T + s];
        REAL ns = -sum;
        for (int64_t v = 0; v < V; v++) br[v] *= ns;
        for (int64_t s = 0; s < T; s++) br[idx[idx_base[r] + s * idx_col_stride]] += g[r * T + s];
    }
}

/* ---------------------------------------------------------------------------------------------
 * Inside forward for one sentence.  calculate_C_kernel (pcfg_loss.cu:262-349) then
 * calculate_S_kernel (pcfg_loss.cu:84-224).  Tables are filled with -inf first (:246, :365).
 * ------------------------------------------------------------------------------------------- */
static void FN(inside_fwd_one)(const REAL *match, const REAL *links, int m, int n, REAL *S, REAL *C,
                               int L, int T, int ml)
{
    const int Mc = (L - 2) / (ml + 1) + 1;
    const int Lc = L - Mc;
    for (size_t i = 0; i < (size_t)Mc * (T + 2); i++) S[i] = NEG_INF;
    for (size_t i = 0; i < (size_t)Lc * (T + 2) * (ml + 2); i++) C[i] = NEG_INF;

    /* pcfg_loss.cu:288-300 */
    C_AT(C, 0, n, 0) = 0;
    for (int i = 0; i < n; i++) C_AT(C, 0, i, 0) = 0;
    for (int a_id = 0; a_id < Lc; a_id++) {
        int a = LT_I2E(a_id);
        int lo = ((a - 1) / (ml + 1)) * (ml + 1) + 1;
        if (a > 0 && a < m && ((a - lo) % 2 == 1))
            for (int i = 0; i < n; i++) C_AT(C, a_id, i, 1) = MA(a, i);
    }
    /* pcfg_loss.cu:301-348 */
    for (int gap = 2; gap < ml + 2; gap++) {
        for (int a_id = 0; a_id < Lc; a_id++) {
            int a = LT_I2E(a_id);
            if (!(a > 0 && a < m)) continue;
            int hi = ((a - 1) / (ml + 1) + 1) * (ml + 1) + 1;
            int b_start = a - ml < 1 ? 1 : a - ml;
            for (int i = 0; i < n - gap - 1; i++) {
                REAL maxval = NEG_INF;
                for (int j = 0; j < gap; j++)
                    for (int b = b_start; b < a + 1; b++) {
                        int _b = b == a ? 0 : b;
                        int b_id = LT_E2I(_b);
                        for (int c = a + 1; c < hi && c < m; c++) {
                            int c_id = LT_E2I(c);
                            REAL t = LK(a, a - b, c) + C_AT(C, b_id, i, j) + C_AT(C, c_id, i + j + 1, gap - j - 1) + MA(a, i + j);
                            if (isnan(t)) t = NEG_INF;
                            if (t > maxval) maxval = t;
                        }
                    }
                REAL res;
                if (isinf(maxval)) {
                    res = maxval;
                } else {
                    REAL sum = 0;
                    for (int j = 0; j < gap; j++)
                        for (int b = b_start; b < a + 1; b++) {
                            int _b = b == a ? 0 : b;
                            int b_id = LT_E2I(_b);
                            for (int c = a + 1; c < hi && c < m; c++) {
                                int c_id = LT_E2I(c);
                                REAL t = LK(a, a - b, c) + C_AT(C, b_id, i, j) + C_AT(C, c_id, i + j + 1, gap - j - 1) + MA(a, i + j) - maxval;
                                if (isnan(t)) t = NEG_INF;
                                sum += EXP(t);
                            }
                        }
                    res = LOG(sum) + maxval;
                }
                C_AT(C, a_id, i, gap) = res;
            }
        }
    }

    /* pcfg_loss.cu:142-147 */
    S_AT(S, MC_E2I(m - 1), n - 1) = MA(m - 1, n - 1);
    /* pcfg_loss.cu:148-214, start = n-2 ... 0 */
    for (int start = n - 2; start >= 0; start--) {
        for (int a_id = 0; a_id < Mc; a_id++) {
            int a = MC_I2E(a_id);
            if (!(a > 0 && a < m)) continue;
            int b_start = a - ml < 1 ? 1 : a - ml;
            REAL maxval = NEG_INF;
            for (int c_id = a_id; MC_I2E(c_id) < m; c_id++) {
                int c = MC_I2E(c_id);
                for (int j = 0; j < n - start && j < ml + 1; j++)
                    for (int b = b_start; b < a + 1; b++) {
                        int _b = b == a ? 0 : b;
                        int b_id = LT_E2I(_b);
                        REAL t = LK(a, a - b, c) + S_AT(S, c_id, start + j + 1) + C_AT(C, b_id, start, j) + MA(a, start + j);
                        if (isnan(t)) t = NEG_INF;
                        if (t > maxval) maxval = t;
                    }
            }
            REAL res;
            if (isinf(maxval)) {
                res = maxval;
            } else {
                REAL sum = 0;
                for (int c_id = a_id; MC_I2E(c_id) < m; c_id++) {
                    int c = MC_I2E(c_id);
                    for (int j = 0; j < n - start && j < ml + 1; j++)
                        for (int b = b_start; b < a + 1; b++) {
                            int _b = b == a ? 0 : b;
                            int b_id = LT_E2I(_b);
                            REAL t = LK(a, a - b, c) + S_AT(S, c_id, start + j + 1) + C_AT(C, b_id, start, j) + MA(a, start + j) - maxval;
                            if (isnan(t)) t = NEG_INF;
                            sum += EXP(t);
                        }
                }
                res = LOG(sum) + maxval;
            }
            S_AT(S, a_id, start) = res;
        }
    }
}

/* Batch driver: pcfg_loss (pcfg_loss.cu:379-401).  S: [B,Mc,T+2], C: [B,Lc,T+2,ml+2]. */
void FN(oracle_inside_fwd)(const REAL *match, const REAL *links, const int64_t *out_len, const int64_t *tgt_len,
                           REAL *S, REAL *C, int B, int L, int T, int ml)
{
    const int Mc = (L - 2) / (ml + 1) + 1;
    const int Lc = L - Mc;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bt = 0; bt < B; bt++)
        FN(inside_fwd_one)(match + (size_t)bt * L * T, links + (size_t)bt * L * (ml + 1) * L, (int)out_len[bt],
                           (int)tgt_len[bt], S + (size_t)bt * Mc * (T + 2), C + (size_t)bt * Lc * (T + 2) * (ml + 2), L, T, ml);
}

/* ---------------------------------------------------------------------------------------------
 * Backward for one sentence: the exact gradient of inside_fwd_one with respect to match and links,
 * organised as the reference's seven kernels (pcfg_loss_backward.cu:28-603).  Sg/Cg are the
 * S_grad/C_grad scratch tables (zero-filled here, :686-687); mg/lg are zero-filled outputs (:689-690).
 * ------------------------------------------------------------------------------------------- */
static void FN(inside_bwd_one)(REAL g, const REAL *S, const REAL *C, const REAL *match, const REAL *links, int m, int n,
                               REAL *Sg, REAL *Cg, REAL *mg, REAL *lg, int L, int T, int ml)
{
    const int Mc = (L - 2) / (ml + 1) + 1;
    const int Lc = L - Mc;
    memset(Sg, 0, sizeof(REAL) * (size_t)Mc * (T + 2));
    memset(Cg, 0, sizeof(REAL) * (size_t)Lc * (T + 2) * (ml + 2));
    memset(mg, 0, sizeof(REAL) * (size_t)L * T);
    memset(lg, 0, sizeof(REAL) * (size_t)L * (ml + 1) * L);
#define MG(a, i) mg[(size_t)(a) * T + (i)]
#define LG(a, k, c) lg[((size_t)(a) * (ml + 1) + (k)) * L + (c)]

    /* calculate_S_kernel_grad, :76-112 (start ascending; exact reading: parents a <= c). */
    S_AT(Sg, 0, 0) = g;
    for (int s = 0; s < n; s++) {
        for (int a_id = 0; a_id < Mc; a_id++) {
            int a = MC_I2E(a_id);
            if (!(a > 0 && a < m)) continue;
            REAL sg = S_AT(Sg, a_id, s), sa = S_AT(S, a_id, s);
            if (sg == 0 || isinf(sa) || isnan(sa)) continue; /* guards :94, :183, :350, :514 */
            int b_start = a - ml < 1 ? 1 : a - ml;
            for (int c_id = a_id; MC_I2E(c_id) < m; c_id++) {
                int c = MC_I2E(c_id);
                for (int j = 0; j < n - s && j < ml + 1; j++) {
                    REAL sc = S_AT(S, c_id, s + j + 1);
                    if (isinf(sc) || isnan(sc)) continue; /* :94 */
                    for (int b = b_start; b < a + 1; b++) {
                        int _b = b == a ? 0 : b;
                        int b_id = LT_E2I(_b);
                        REAL t = LK(a, a - b, c) + sc + C_AT(C, b_id, s, j) + MA(a, s + j) - sa;
                        if (isnan(t) || t == NEG_INF) continue;
                        REAL p = sg * EXP(t);
                        S_AT(Sg, c_id, s + j + 1) += p;      /* :109 */
                        if (b_id != 0) C_AT(Cg, b_id, s, j) += p; /* calculate_C_kernel_grad_1 :190-203 */
                        MG(a, s + j) += p;                    /* calculate_match_all_kernel_grad_1 :361-374 */
                        LG(a, a - b, c) += p;                 /* calculate_links_kernel_grad_1 :525-528 */
                    }
                }
            }
        }
    }
    /* :379-382 */
    MG(m - 1, n - 1) += S_AT(Sg, MC_E2I(m - 1), n - 1);

    /* Local trees, gap descending (calculate_C_kernel_grad_2 :236-276, calculate_match_all_kernel_grad_2
     * :407-428, calculate_links_kernel_grad_2 :556-599), exact reading with the forward's ranges. */
    for (int gap = ml + 1; gap >= 2; gap--) {
        for (int a_id = 0; a_id < Lc; a_id++) {
            int a = LT_I2E(a_id);
            if (!(a > 0 && a < m)) continue;
            int hi = ((a - 1) / (ml + 1) + 1) * (ml + 1) + 1;
            int b_start = a - ml < 1 ? 1 : a - ml;
            for (int i = 0; i < n - gap - 1; i++) {
                REAL cg = C_AT(Cg, a_id, i, gap), ca = C_AT(C, a_id, i, gap);
                if (cg == 0 || isinf(ca) || isnan(ca)) continue;
                for (int j = 0; j < gap; j++)
                    for (int b = b_start; b < a + 1; b++) {
                        int _b = b == a ? 0 : b;
                        int b_id = LT_E2I(_b);
                        for (int c = a + 1; c < hi && c < m; c++) {
                            int c_id = LT_E2I(c);
                            REAL t = LK(a, a - b, c) + C_AT(C, b_id, i, j) + C_AT(C, c_id, i + j + 1, gap - j - 1) + MA(a, i + j) - ca;
                            if (isnan(t) || t == NEG_INF) continue;
                            REAL p = cg * EXP(t);
                            if (b_id != 0) C_AT(Cg, b_id, i, j) += p;
                            C_AT(Cg, c_id, i + j + 1, gap - j - 1) += p;
                            MG(a, i + j) += p;
                            LG(a, a - b, c) += p;
                        }
                    }
            }
        }
    }
    /* leaves, :429-433 */
    for (int a_id = 0; a_id < Lc; a_id++) {
        int a = LT_I2E(a_id);
        int lo = ((a - 1) / (ml + 1)) * (ml + 1) + 1;
        if (a > 0 && a < m && ((a - lo) % 2 == 1))
            for (int i = 0; i < n; i++) MG(a, i) += C_AT(Cg, a_id, i, 1);
    }
#undef MG
#undef LG
}

/* pcfg_loss_backward (pcfg_loss_backward.cu:654-721).  Sg/Cg are caller-provided scratch of the
 * same shapes as S/C. */
void FN(oracle_inside_bwd)(const REAL *grad_out, const REAL *S, const REAL *C, const REAL *match, const REAL *links,
                           const int64_t *out_len, const int64_t *tgt_len, REAL *Sg, REAL *Cg, REAL *mg, REAL *lg,
                           int B, int L, int T, int ml)
{
    const int Mc = (L - 2) / (ml + 1) + 1;
    const int Lc = L - Mc;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bt = 0; bt < B; bt++) {
        size_t so = (size_t)bt * Mc * (T + 2), co = (size_t)bt * Lc * (T + 2) * (ml + 2);
        FN(inside_bwd_one)(grad_out[bt], S + so, C + co, match + (size_t)bt * L * T, links + (size_t)bt * L * (ml + 1) * L,
                           (int)out_len[bt], (int)tgt_len[bt], Sg + so, Cg + co, mg + (size_t)bt * L * T,
                           lg + (size_t)bt * L * (ml + 1) * L, L, T, ml);
    }
}

/* ---------------------------------------------------------------------------------------------
 * Best tree for one sentence: calculate_S_trace_kernel (pcfg_best_tree.cu:64-197) then
 * calculate_C_kernel_trace (:239-301).  The 4-lane scan and the strict-'>' lane merge
 * (lane priority 0 > 2 > 1 > 3, :140-174) are reproduced so that exact ties resolve identically.
 * St/Ct: zero-filled mark tables shaped like S/C.  tree: [L] int64, filled with -1 (:220).
 * min_margin (may be NULL; not part of the reference): three values about the arg-max decisions of the trace that had
 * two finite candidates - [0] the smallest gap between the best and the second-best candidate (0 = exact tie, +inf = no
 * such decision), [1] the number of exact ties, [2] the smallest gap that is not a tie: how far the chosen indices are
 * from flipping under rounding, and how often only the scan order decides.
 * ------------------------------------------------------------------------------------------- */
#define TRACK_MARGIN(t)                                \
    do {                                               \
        if ((t) > g1) { g2 = g1; g1 = (t); }           \
        else if ((t) > g2) g2 = (t);                   \
    } while (0)
#define CLOSE_MARGIN()                                                                                   \
    do {                                                                                                 \
        if (min_margin && g2 > NEG_INF) {                                                                \
            REAL gap_ = g1 - g2;                                                                         \
            if (gap_ < min_margin[0]) min_margin[0] = gap_;                                              \
            if (gap_ == 0) min_margin[1] += 1;                                                           \
            else if (gap_ < min_margin[2]) min_margin[2] = gap_;                                         \
        }                                                                                                \
    } while (0)
static void FN(best_tree_one)(const REAL *S, const REAL *C, const REAL *match, const REAL *links, int m, int n,
                              unsigned char *St, unsigned char *Ct, int64_t *tree, int L, int T, int ml, REAL *min_margin)
{
    const int Mc = (L - 2) / (ml + 1) + 1;
    const int Lc = L - Mc;
    memset(St, 0, (size_t)Mc * (T + 2));
    memset(Ct, 0, (size_t)Lc * (T + 2) * (ml + 2));
    for (int a = 0; a < L; a++) tree[a] = -1;
    if (min_margin) { min_margin[0] = min_margin[2] = -NEG_INF; min_margin[1] = 0; }
    S_AT(St, 0, 0) = 1; /* :112-116 */
    for (int s = 0; s <= n; s++) { /* task index start-1, :94-119 */
        for (int a_id = 0; a_id < Mc; a_id++) {
            int a = MC_I2E(a_id);
            if (!(a > 0 && a < m && S_AT(St, a_id, s) != 0)) continue;
            int b_start = a - ml < 1 ? 1 : a - ml;
            REAL lane_val[4];
            int lane_c[4], lane_j[4], lane_b[4];
            REAL g1 = NEG_INF, g2 = NEG_INF;
            for (int x = 0; x < 4; x++) {
                REAL maxval = NEG_INF;
                int max_c = -1, max_j = 0, max_b = -1;
                for (int c_id = a_id + x + 1; MC_I2E(c_id) < m; c_id += 4) { /* :123 */
                    int c = MC_I2E(c_id);
                    for (int j = 0; j < n - s && j < ml + 1; j++)
                        for (int b = b_start; b < a + 1; b++) {
                            int _b = b == a ? 0 : b;
                            int b_id = LT_E2I(_b);
                            REAL t = LK(a, a - b, c) + S_AT(S, c_id, s + j + 1) + C_AT(C, b_id, s, j) + MA(a, s + j);
                            if (isnan(t)) t = NEG_INF;
                            TRACK_MARGIN(t);
                            if (t > maxval) { maxval = t; max_c = c_id; max_j = j; max_b = b_id; }
                        }
                }
                lane_val[x] = maxval; lane_c[x] = max_c; lane_j[x] = max_j; lane_b[x] = max_b;
            }
            /* shfl_down 2 then 1 with strict '>' (:159-170) */
            for (int x = 0; x < 2; x++)
                if (lane_val[x + 2] > lane_val[x]) { lane_val[x] = lane_val[x + 2]; lane_c[x] = lane_c[x + 2]; lane_j[x] = lane_j[x + 2]; lane_b[x] = lane_b[x + 2]; }
            if (lane_val[1] > lane_val[0]) { lane_val[0] = lane_val[1]; lane_c[0] = lane_c[1]; lane_j[0] = lane_j[1]; lane_b[0] = lane_b[1]; }
            if (lane_c[0] != -1 && lane_b[0] != -1) { /* :178-181 */
                S_AT(St, lane_c[0], s + lane_j[0] + 1) = 1;
                C_AT(Ct, lane_b[0], s, lane_j[0]) = 1;
            }
            tree[a] = s + lane_j[0]; /* :182 */
            CLOSE_MARGIN();
        }
    }
    if (ml == 0) return; /* :308 */
    for (int gap = ml + 1; gap >= 1; gap--) { /* :268-300 */
        for (int a_id = 1; a_id < Lc; a_id++) {
            int a = LT_I2E(a_id);
            if (!(a > 0 && a < m)) continue;
            int hi = ((a - 1) / (ml + 1) + 1) * (ml + 1) + 1;
            int b_start = a - ml < 1 ? 1 : a - ml;
            for (int i = 0; i < n - gap - 1; i++) {
                if (C_AT(Ct, a_id, i, gap) == 0) continue;
                int max_j = 0, max_b = -1, max_c = -1;
                REAL maxval = NEG_INF, g1 = NEG_INF, g2 = NEG_INF;
                for (int j = 0; j < gap; j++)
                    for (int b = b_start; b < a + 1; b++) {
                        int _b = b == a ? 0 : b;
                        int b_id = LT_E2I(_b);
                        for (int c = a + 1; c < hi && c < m; c++) {
                            int c_id = LT_E2I(c);
                            REAL t = LK(a, a - b, c) + C_AT(C, b_id, i, j) + C_AT(C, c_id, i + j + 1, gap - j - 1) + MA(a, i + j);
                            if (isnan(t)) t = NEG_INF;
                            TRACK_MARGIN(t);
                            if (t > maxval) { maxval = t; max_j = j; max_b = b_id; max_c = c_id; }
                        }
                    }
                CLOSE_MARGIN();
                if (max_b != -1 && max_c != -1) {
                    C_AT(Ct, max_b, i, max_j) = 1;
                    C_AT(Ct, max_c, i + max_j + 1, gap - max_j - 1) = 1;
                }
                tree[a] = i + max_j;
            }
        }
    }
}

/* pcfg_best_tree (pcfg_best_tree.cu:333-360). */
void FN(oracle_best_tree)(const REAL *S, const REAL *C, const REAL *match, const REAL *links, const int64_t *out_len,
                          const int64_t *tgt_len, int64_t *tree, REAL *min_margin, int B, int L, int T, int ml)
{
    const int Mc = (L - 2) / (ml + 1) + 1;
    const int Lc = L - Mc;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bt = 0; bt < B; bt++) {
        unsigned char *St = (unsigned char *)malloc((size_t)Mc * (T + 2));
        unsigned char *Ct = (unsigned char *)malloc((size_t)Lc * (T + 2) * (ml + 2));
        FN(best_tree_one)(S + (size_t)bt * Mc * (T + 2), C + (size_t)bt * Lc * (T + 2) * (ml + 2), match + (size_t)bt * L * T,
                          links + (size_t)bt * L * (ml + 1) * L, (int)out_len[bt], (int)tgt_len[bt], St, Ct,
                          tree + (size_t)bt * L, L, T, ml, min_margin ? min_margin + 3 * bt : NULL);
        free(St);
        free(Ct);
    }
}

/* ---------------------------------------------------------------------------------------------
 * Viterbi tables for one sentence: calculate_C_kernel (pcfg_viterbi.cu:177-241) then
 * calculate_S_kernel (:22-140).  Tables [L, Lq] with Lq = L/4, indexed by external node id.
 * S, Cv initialised to -inf (:159, :256), traces to 0 (:287-289).  The additions keep the
 * reference's left-to-right order so that fp32 values - and therefore arg-max decisions - are
 * reproducible bit for bit.
 * ------------------------------------------------------------------------------------------- */
static void FN(viterbi_one)(const REAL *ob, const REAL *links, int m, REAL *S, REAL *Cv, int64_t *R, int64_t *Lt,
                            int64_t *M, int L, int ml, REAL *min_margin)
{
    const int Lq = L / 4;
    if (min_margin) { min_margin[0] = min_margin[2] = -NEG_INF; min_margin[1] = 0; } /* as in best_tree_one, over every table entry */
#define V_AT(t, a, l) (t)[(size_t)(a) * Lq + (l)]
    for (size_t i = 0; i < (size_t)L * Lq; i++) { S[i] = NEG_INF; Cv[i] = NEG_INF; R[i] = 0; Lt[i] = 0; M[i] = 0; }
    for (int a = 1; a < L; a++) { /* :196-205 */
        int lo = ((a - 1) / (ml + 1)) * (ml + 1) + 1;
        if (a > 0 && a < m && ((a - lo) % 2 == 1)) V_AT(Cv, a, 1) = ob[a];
    }
    V_AT(Cv, 0, 0) = 0; /* :206-208 */
    for (int gap = 2; gap < ml + 1; gap++) { /* :214-237 */
        for (int a = 1; a < L; a++) {
            if (!(a > 0 && a < m && (a % (ml + 1) != 1))) continue;
            int hi = ((a - 1) / (ml + 1) + 1) * (ml + 1) + 1;
            int b_start = a - ml < 1 ? 1 : a - ml;
            REAL maxval = NEG_INF, g1 = NEG_INF, g2 = NEG_INF;
            int max_b = 0, max_c = 0, max_j = 0;
            for (int j = 0; j < gap; j++)
                for (int b = b_start; b < a + 1; b++) {
                    int _b = b == a ? 0 : b;
                    for (int c = a + 1; c < hi && c < m; c++) {
                        REAL t = LK(a, a - b, c) + V_AT(Cv, _b, j) + V_AT(Cv, c, gap - j - 1) + ob[a];
                        if (isnan(t)) t = NEG_INF;
                        TRACK_MARGIN(t);
                        if (t > maxval) { maxval = t; max_b = _b; max_c = c; max_j = j; }
                    }
                }
            CLOSE_MARGIN();
            if (!isinf(maxval)) {
                V_AT(Cv, a, gap) = maxval; V_AT(R, a, gap) = max_c; V_AT(Lt, a, gap) = max_b; V_AT(M, a, gap) = max_j;
            }
        }
    }
    V_AT(S, m - 1, 1) = ob[m - 1]; /* :57-59 */
    for (int len = 2; len < m / 4; len++) { /* :67 */
        for (int id = 0; id * (ml + 1) + 1 < m; id++) {
            int a = id * (ml + 1) + 1;
            int b_start = a - ml < 1 ? 1 : a - ml;
            REAL lane_val[4];
            int lane_c[4], lane_j[4], lane_b[4];
            REAL g1 = NEG_INF, g2 = NEG_INF;
            for (int x = 0; x < 4; x++) {
                REAL maxval = NEG_INF;
                int max_b = 0, max_c = 0, max_j = 0;
                for (int c_id = id + x; c_id * (ml + 1) + 1 < m; c_id += 4) { /* :75 */
                    int c = c_id * (ml + 1) + 1;
                    for (int j = 0; j < ml + 1; j++)
                        for (int b = b_start; b < a + 1; b++) {
                            int _b = b == a ? 0 : b;
                            REAL sc = (len - j - 1 >= 0) ? V_AT(S, c, len - j - 1) : NEG_INF;
                            REAL t = LK(a, a - b, c) + V_AT(Cv, _b, j) + sc + ob[a]; /* :83 */
                            if (isnan(t)) t = NEG_INF;
                            TRACK_MARGIN(t);
                            if (t > maxval) { maxval = t; max_b = _b; max_c = c; max_j = j; }
                        }
                }
                lane_val[x] = maxval; lane_c[x] = max_c; lane_j[x] = max_j; lane_b[x] = max_b;
            }
            for (int x = 0; x < 2; x++) /* :109-120 */
                if (lane_val[x + 2] > lane_val[x]) { lane_val[x] = lane_val[x + 2]; lane_c[x] = lane_c[x + 2]; lane_j[x] = lane_j[x + 2]; lane_b[x] = lane_b[x + 2]; }
            if (lane_val[1] > lane_val[0]) { lane_val[0] = lane_val[1]; lane_c[0] = lane_c[1]; lane_j[0] = lane_j[1]; lane_b[0] = lane_b[1]; }
            if (!isinf(lane_val[0])) { /* :125-131 */
                V_AT(S, a, len) = lane_val[0]; V_AT(Lt, a, len) = lane_b[0]; V_AT(R, a, len) = lane_c[0]; V_AT(M, a, len) = lane_j[0];
            }
            CLOSE_MARGIN();
        }
    }
#undef V_AT
}

/* pcfg_viterbi (pcfg_viterbi.cu:272-301).  S: [B,L,Lq] (the wrapper returns row 1), Cv: scratch of the
 * same shape, R/Lt/M: [B,L,Lq] int64. */
void FN(oracle_viterbi)(const REAL *ob, const REAL *links, const int64_t *out_len, REAL *S, REAL *Cv, int64_t *R, int64_t *Lt,
                        int64_t *M, REAL *min_margin, int B, int L, int ml)
{
    const int Lq = L / 4;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bt = 0; bt < B; bt++) {
        size_t o = (size_t)bt * L * Lq;
        FN(viterbi_one)(ob + (size_t)bt * L, links + (size_t)bt * L * (ml + 1) * L, (int)out_len[bt], S + o, Cv + o, R + o, Lt + o,
                        M + o, L, ml, min_margin ? min_margin + 3 * bt : NULL);
    }
}

#undef TRACK_MARGIN
#undef CLOSE_MARGIN
#undef MC_I2E
#undef MC_E2I
#undef LT_I2E
#undef LT_E2I
#undef S_AT
#undef C_AT
#undef LK
#undef MA
#undef NEG_INF
