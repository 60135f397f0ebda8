// The part of the GLAT pass that follows the best-tree alignment (reference fs_plugins/criterions/nat_pcfg_loss.py:216-255):
// path clipping, match mask, oracle tokens, number of correct predictions, glance threshold, revealed tokens - the work
// of one workgroup per sentence, as a block that a kernel of its own runs or the kernel that has just walked the tree.
#pragma once
#include "common.hip.h"

namespace pcfgnat {

struct GlatGlueArgs {
    int64_t *path;                 // [B,L]: the alignment on entry (-1 = node off the tree), the clipped path on exit (:217-218)
    const int64_t *targets;        // [B,T]
    const int64_t *prev_tokens;    // [B,L]
    const int64_t *pred_tokens;    // [B,L]
    const float *noise;            // [B,L]  (number-random, cmlm)
    const float *length_rand;      // [B]    (cmlm)
    const float *keep_rand;        // [B,L]  (default strategy)
    int strategy;
    const int64_t *lengths;        // [2,B]: graph lengths, target lengths
    float context_p;
    unsigned char *matchmask;      // [B,T,L]
    unsigned char *keep_mask;      // [B,L]
    int64_t *glat_tokens;          // [B,L]
    int64_t *same_num, *glance_nums;  // [B]
    int B, L, T;
    LossTask loss;
};

// The best tree of every sentence (max_left = 1) and this glue behind it in one launch; g.path receives the tree (inside.hip).
int best_tree_glue_ml1(const float *S, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, int64_t B,
                       int64_t L, int64_t T, const GlatGlueArgs &glue, void *stream);

// What the glue reads that does not depend on the alignment, for the thread's first node (node threadIdx.x, if the graph
// has one): requested ahead of the tree walk by the kernel that does both, so that it has arrived when the walk ends.
struct GlatGlueEarly {
    int64_t pred, prev;
    float draw;  // the node's noise value (number-random, cmlm) or its uniform draw (default strategy)
};
__device__ __forceinline__ GlatGlueEarly glat_glue_early(const int b, const GlatGlueArgs &g) {
    const int a = threadIdx.x;
    const size_t o = (size_t)b * g.L + (a < g.L ? a : 0);
    GlatGlueEarly e;
    e.pred = g.pred_tokens[o];
    e.prev = g.prev_tokens[o];
    e.draw = (g.strategy == PCFGNAT_GLANCE_DEFAULT ? g.keep_rand : g.noise)[o];
    return e;
}

// Sentence b by a workgroup of NT threads, all of which must call it.  dyn: 2 L floats of LDS (prob [L] float, path [L] int).
// early, raw_lds ([L]: the alignment as the walk left it) and tg_lds ([T]: the sentence's targets) may be null: the block
// then reads all of it from global memory.
template <int NT>
__device__ __forceinline__ void glat_glue_block(const int b, const GlatGlueArgs &g, float *dyn, const GlatGlueEarly *early = nullptr,
                                                const int *raw_lds = nullptr, const int64_t *tg_lds = nullptr) {
    const int B = g.B, L = g.L, T = g.T, strategy = g.strategy;
    int64_t *__restrict__ path = g.path;
    const int64_t *__restrict__ pred_tokens = g.pred_tokens, *__restrict__ prev_tokens = g.prev_tokens;
    const float *__restrict__ noise = g.noise, *__restrict__ keep_rand = g.keep_rand;
    unsigned char *__restrict__ keep_mask = g.keep_mask;
    int64_t *__restrict__ glat_tokens = g.glat_tokens;
    const float context_p = g.context_p;
    float *s_prob = dyn;                              // [L]
    int *s_path = reinterpret_cast<int *>(dyn + L);   // [L]
    __shared__ int s_same;
    __shared__ float s_thresh;
    const int tid = threadIdx.x;
    if (g.loss.out != nullptr && b == 0) criterion_loss_block<256, NT>(g.loss);  // -(ll/n).mean() over the valid sentences (:212-214, 268)
    const int64_t n = g.lengths[(size_t)B + b];
    const int64_t *tg = tg_lds != nullptr ? tg_lds : g.targets + (size_t)b * T;
    if (tid == 0) {
        s_same = 0;
        s_thresh = 100.f;
    }
    __syncthreads();
    int same = 0;
    for (int a = tid; a < L; a += NT) {
        const bool first = early != nullptr && a == tid;   // the node whose inputs came early
        const int64_t raw = raw_lds != nullptr ? (int64_t)raw_lds[a] : path[(size_t)b * L + a];
        const bool align = raw >= 0;                       // predict_align_mask (:216), taken before the clipping
        int64_t p = raw;
        if (p + 1 >= (int64_t)T + 1) p = -1;               // :217
        if (p + 1 < 0) p = -1;                             // :218
        path[(size_t)b * L + a] = p;
        s_path[a] = (int)p;
        const int64_t oracle = tg[p < 0 ? 0 : p];          // :227
        same += ((first ? early->pred : pred_tokens[(size_t)b * L + a]) == oracle) && align;  // :230
        // number-random and cmlm: the glance scores (:235-236, 245-246); default strategy: the alignment mask itself
        s_prob[a] = strategy == PCFGNAT_GLANCE_DEFAULT ? (align ? 1.f : 0.f)
                                                        : (align ? (first ? early->draw : noise[(size_t)b * L + a]) : -100.f);
    }
    same = (int)wave_sum((float)same);
    if ((tid & 63) == 0) atomicAdd(&s_same, same);
    __syncthreads();
    const int total_same = s_same;
    // glance_nums = ((target_length - same_num) * context_p + 0.5).to(long) in float32 (:237); cmlm: a uniform fraction of
    // the target length instead (:247); the default strategy has none
    const int64_t glance = strategy == PCFGNAT_GLANCE_CMLM      ? (int64_t)((float)n * g.length_rand[b] + 0.5f)
                           : strategy == PCFGNAT_GLANCE_DEFAULT ? 0
                                                                : (int64_t)((float)(n - total_same) * context_p + 0.5f);
    if (tid == 0) {
        g.same_num[b] = total_same;
        g.glance_nums[b] = glance;
    }
    // match mask [T][L]: node a carries target position t (:225)
    unsigned char *mm = g.matchmask + (size_t)b * T * L;
    if ((L & 3) == 0 && (reinterpret_cast<uintptr_t>(mm) & 3) == 0) {  // four nodes per store
        uchar4 *mm4 = reinterpret_cast<uchar4 *>(mm);
        for (int i = tid; i < T * L / 4; i += NT) {
            const int t = (4 * i) / L, a = 4 * i - t * L;
            mm4[i] = make_uchar4(s_path[a] == t, s_path[a + 1] == t, s_path[a + 2] == t, s_path[a + 3] == t);
        }
    } else {
        for (int i = tid; i < T * L; i += NT) {
            const int t = i / L, a = i - t * L;
            mm[i] = s_path[a] == t;
        }
    }
    // threshold = the glance-th largest noise value (:238-240); every thread ranks its own values
    if (glance != 0 && strategy != PCFGNAT_GLANCE_DEFAULT) {
        const int64_t k = (glance - 1 < 0) ? 0 : (glance - 1 >= L ? L - 1 : glance - 1);  // index into the descending order
        // PARTS neighbouring lanes share a node's comparisons (a power of two, so that their counts meet by lane exchanges)
        int parts = 1;
        while (parts < 64 && 2 * parts * L <= NT) parts *= 2;
        const int sub = tid & (parts - 1);
        for (int a0 = 0; a0 < L; a0 += NT / parts) {  // (uniform trip count: the exchanges need every lane)
            const int a = a0 + tid / parts;
            const float v = s_prob[a < L ? a : 0];
            int gt = 0, ge = 0;
            for (int o = sub; o < L; o += parts) {
                const float w = s_prob[o];
                gt += w > v;
                ge += w >= v;
            }
            for (int x = 1; x < parts; x *= 2) {
                gt += __shfl_xor(gt, x);
                ge += __shfl_xor(ge, x);
            }
            if (a < L && gt <= k && k < ge) s_thresh = v;  // all writers hold the same value
        }
    }
    __syncthreads();
    const float thresh = s_thresh;
    // default strategy (:231-233): every aligned node is revealed with probability (n - same) / n * context_p, in float32
    const float share = (float)(n - total_same) / (float)n * context_p;
    for (int a = tid; a < L; a += NT) {
        // number-random, cmlm: keep_prob is 0 or 1 and the uniform draw lies in [0, 1): rand < keep_prob is keep_prob
        // itself (:241, 253)
        const bool first = early != nullptr && a == tid;
        const bool keep = strategy == PCFGNAT_GLANCE_DEFAULT ? (first ? early->draw : keep_rand[(size_t)b * L + a]) < share * s_prob[a]
                                                             : s_prob[a] >= thresh;
        const int p = s_path[a];
        keep_mask[(size_t)b * L + a] = keep;
        glat_tokens[(size_t)b * L + a] = keep ? tg[p < 0 ? 0 : p] : (first ? early->prev : prev_tokens[(size_t)b * L + a]);  // :255
    }
}

}  // namespace pcfgnat
