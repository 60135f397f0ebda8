/*
 * TEST INFRASTRUCTURE ONLY.  CPU oracle for the PCFG-NAT structured-loss path: instantiates
 * pcfg_oracle_body.h for float and double and adds the integer-only tree-to-sequence readout.
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -shared).  Loaded through ctypes by oracle/oracle.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define REAL float
#define FN(name) name##_f32
#define EXP expf
#define LOG logf
#include "pcfg_oracle_body.h"
#undef REAL
#undef FN
#undef EXP
#undef LOG

#define REAL double
#define FN(name) name##_f64
#define EXP exp
#define LOG log
#include "pcfg_oracle_body.h"
#undef REAL
#undef FN
#undef EXP
#undef LOG

/* Number of OpenMP threads the batch loops will use (1 when built without OpenMP). */
int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/*
 * viterbi_decoding (pcfg_loss.cpp:12-73): explicit-stack in-order walk of the (L, R, M) traces.
 * Lt/R/M: [B, L, Lq] int64; tokens: [B, L] int64; left_mask: [mask_dim, mask_dim] int64 (1 = forbidden);
 * out: [B, cap] int64 receives the emitted tokens of each sentence, out_len[B] their count.
 * A sentence that would emit more than `cap` tokens has out_len set to -1.
 * The reference then right-pads every row with pad_index to the longest row and returns float32 (:65);
 * that packing is done by the Python wrapper.
 */
void oracle_viterbi_decoding(const int64_t *pred_len, const int64_t *out_length, const int64_t *Lt, const int64_t *R,
                             const int64_t *M, const int64_t *tokens, const int64_t *left_mask, int64_t mask_dim,
                             int64_t pad_index, int64_t *out, int64_t *out_len, int B, int L, int Lq, int cap)
{
    for (int i = 0; i < B; i++) {
        const int64_t *Li = Lt + (size_t)i * L * Lq, *Ri = R + (size_t)i * L * Lq, *Mi = M + (size_t)i * L * Lq;
        int64_t *stack_node = (int64_t *)malloc(sizeof(int64_t) * (size_t)(2 * L + 4));
        int64_t *stack_len = (int64_t *)malloc(sizeof(int64_t) * (size_t)(2 * L + 4));
        int sp = 0, cnt = 0, overflow = 0;
        int64_t node = 1, len = pred_len[i]; /* :26-27 */
        int64_t max_h = out_length[i];       /* :30 */
        int64_t last = -1;
        while ((node < max_h && node != 0) || sp > 0) { /* :32 */
            while (node < max_h && node != 0) {         /* :34 */
                if (sp >= 2 * L + 4) { overflow = 1; break; }
                stack_node[sp] = node; stack_len[sp] = len; sp++;
                int64_t l = Li[(size_t)node * Lq + len]; /* :37 */
                l = (l == node) ? 0 : l;                 /* :38 */
                if (left_mask[(size_t)node * mask_dim + l]) break; /* :39-42 */
                int64_t nl = Mi[(size_t)node * Lq + len];          /* :43 */
                node = l; len = nl;
            }
            if (overflow) break;
            sp--; node = stack_node[sp]; len = stack_len[sp]; /* :46-47 */
            int64_t tok = tokens[(size_t)i * L + node];       /* :48 */
            if (tok != pad_index && tok != last) {            /* :49-53 */
                last = tok;
                if (cnt < cap) out[(size_t)i * cap + cnt] = tok; else overflow = 1;
                cnt++;
            }
            int64_t r = Ri[(size_t)node * Lq + len];                  /* :54 */
            int64_t nl = len - Mi[(size_t)node * Lq + len] - 1;       /* :55 */
            node = r; len = nl;
            if (len < 0 || len >= Lq) { if (node < max_h && node != 0) { overflow = 1; break; } }
        }
        out_len[i] = overflow ? -1 : cnt;
        free(stack_node);
        free(stack_len);
    }
}


/*
 * `lookahead` / `greedy` decode (glat_decomposed_with_link_two_hands_tri_pcfg.py:419-481).
 *
 * Pointers (:420-431): links_idx[b][a] = first arg max over the flattened (k, c) of
 *   lookahead: (links[b][a][k][c] + ob[b][c] * beta) + ob[b][left(a,k)] * beta,  left(a,0) = 0, left(a,k) = max(a-k, 0)
 *              (the `_max_left_index` table, :214-218), each product and sum rounded to fp32 in this order;
 *   greedy (ob == NULL): links[b][a][k][c].
 * The reference builds the left term from `unreduced_logits.unsqueeze(1).repeat(bsz, prelen, 1)` gathered with a
 * batch-1 index (:424), which for bsz > 1 takes sentence 0's logits for every sentence; like its viterbi_decoding it is
 * effectively a batch-1 routine, and the evidently intended per-sentence term is used here.
 * Walk (:434-476): in-order traversal from node 1: descend to the left child (0 if k = 0, else a - k) unless
 * left_mask[a][left] is set, emit tokens[a] unless it is the pad symbol, continue with the right child c; stop when the
 * stack is empty and the current node is 0 or >= output_length.  No de-duplication (unlike viterbi_decoding).
 * out [B][cap], out_len [B] (-1 if the walk does not terminate within the cell budget).
 */
void oracle_lookahead_decode(const float *links, const float *ob, float beta, const int64_t *out_length, const int64_t *tokens,
                             const int64_t *left_mask, int64_t mask_dim, int64_t pad_index, int64_t *links_idx, int64_t *out,
                             int64_t *out_len, int B, int L, int ml, int cap)
{
    const int K = ml + 1;
    for (int b = 0; b < B; b++) {
        const float *lk = links + (size_t)b * L * K * L;
        for (int a = 0; a < L; a++) {
            float best = 0.f;
            int best_i = -1;
            for (int k = 0; k < K; k++) {
                const int left = (k == 0) ? 0 : (a - k < 0 ? 0 : a - k);
                for (int c = 0; c < L; c++) {
                    float v = lk[((size_t)a * K + k) * L + c];
                    if (ob) {
                        const float r = ob[(size_t)b * L + c] * beta;
                        const float l = ob[(size_t)b * L + left] * beta;
                        v = (v + r) + l;
                    }
                    if (best_i < 0 || v > best) { best = v; best_i = k * L + c; }
                }
            }
            links_idx[(size_t)b * L + a] = best_i;
        }
        int64_t *stack = (int64_t *)malloc(sizeof(int64_t) * (size_t)(L + 4));
        int sp = 0, cnt = 0, bad = 0;
        int64_t now = 1, length = out_length[b];
        int64_t budget = 4 * (int64_t)L + 8;
        while ((now < length && now != 0) || sp > 0) {
            if (--budget < 0) { bad = 1; break; }
            while (now < length && now != 0) {
                if (sp >= L + 4 || now < 0 || now >= L) { bad = 1; break; }
                stack[sp++] = now;
                const int64_t k = links_idx[(size_t)b * L + now] / L;
                const int64_t left = (k == 0) ? 0 : now - k;
                if (left < 0 || left >= mask_dim || now >= mask_dim) { bad = 1; break; }
                if (left_mask[(size_t)now * mask_dim + left]) break;
                now = left;
            }
            if (bad) break;
            now = stack[--sp];
            const int64_t tok = tokens[(size_t)b * L + now];
            if (tok != pad_index) {
                if (cnt < cap) out[(size_t)b * cap + cnt] = tok; else bad = 1;
                cnt++;
            }
            now = links_idx[(size_t)b * L + now] % L;
        }
        out_len[b] = bad ? -1 : cnt;
        free(stack);
    }
}
