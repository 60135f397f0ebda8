// GLAT glancing (reference fs_plugins/criterions/nat_pcfg_loss.py:193-269, all three glance strategies: :231-233 the
// default, :235-242 `number-random`, :244-251 `cmlm`) as one native
// call: sentence lengths from the pad counts, fused log-softmax + gather + eos mask + arg max in one read of the logits,
// inside forward, best-tree alignment, and one small kernel per sentence for everything the criterion does with the
// alignment (path clipping, match mask, oracle tokens, number of correct predictions, glance threshold, revealed
// tokens).  The random numbers of the sampling step are drawn by the caller with its own generator, in the reference's
// order, so that the random stream is the one the torch code consumes.
#include "common.hip.h"

namespace pcfgnat {
namespace {

constexpr int GNT = 256;

// lengths[0][b] = number of non-pad decoder inputs (nat_pcfg_loss.py:196), lengths[1][b] = non-pad targets (:195)
__global__ __launch_bounds__(GNT) void glat_lengths_kernel(const int64_t *__restrict__ prev_tokens, const int64_t *__restrict__ targets,
                                                          int64_t pad, int64_t *__restrict__ lengths, int B, int L, int T) {
    __shared__ int s_cnt[2];
    const int b = blockIdx.x, tid = threadIdx.x;
    if (tid < 2) s_cnt[tid] = 0;
    __syncthreads();
    int c0 = 0, c1 = 0;
    for (int i = tid; i < L; i += GNT) c0 += prev_tokens[(size_t)b * L + i] != pad;
    for (int i = tid; i < T; i += GNT) c1 += targets[(size_t)b * T + i] != pad;
    c0 = (int)wave_sum((float)c0);
    c1 = (int)wave_sum((float)c1);
    if ((tid & 63) == 0) {
        atomicAdd(&s_cnt[0], c0);
        atomicAdd(&s_cnt[1], c1);
    }
    __syncthreads();
    if (tid == 0) {
        lengths[b] = s_cnt[0];
        lengths[(size_t)B + b] = s_cnt[1];
    }
}

// One workgroup per sentence.  `path` holds the best-tree alignment on entry (-1 = node off the tree) and the clipped
// path on exit (:217-218).  Dynamic LDS: prob [L] float, path [L] int.
__global__ __launch_bounds__(GNT) void glat_glue_kernel(int64_t *__restrict__ path, const int64_t *__restrict__ targets,
                                                       const int64_t *__restrict__ prev_tokens, const int64_t *__restrict__ pred_tokens,
                                                       const float *__restrict__ noise, const float *__restrict__ length_rand,
                                                       const float *__restrict__ keep_rand, int strategy,
                                                       const int64_t *__restrict__ lengths, float context_p,
                                                       unsigned char *__restrict__ matchmask,
                                                       unsigned char *__restrict__ keep_mask, int64_t *__restrict__ glat_tokens,
                                                       int64_t *__restrict__ same_num, int64_t *__restrict__ glance_nums, int B, int L,
                                                       int T, LossTask loss) {
    extern __shared__ float dyn[];
    float *s_prob = dyn;                              // [L]
    int *s_path = reinterpret_cast<int *>(dyn + L);   // [L]
    __shared__ int s_same;
    __shared__ float s_thresh;
    const int b = blockIdx.x, tid = threadIdx.x;
    if (loss.out != nullptr && b == 0) criterion_loss_block<GNT>(loss);  // -(ll/n).mean() over the valid sentences (:212-214, 268)
    const int64_t n = lengths[(size_t)B + b];
    const int64_t *tg = targets + (size_t)b * T;
    if (tid == 0) {
        s_same = 0;
        s_thresh = 100.f;
    }
    __syncthreads();
    int same = 0;
    for (int a = tid; a < L; a += GNT) {
        const int64_t raw = path[(size_t)b * L + a];
        const bool align = raw >= 0;                       // predict_align_mask (:216), taken before the clipping
        int64_t p = raw;
        if (p + 1 >= (int64_t)T + 1) p = -1;               // :217
        if (p + 1 < 0) p = -1;                             // :218
        path[(size_t)b * L + a] = p;
        s_path[a] = (int)p;
        const int64_t oracle = tg[p < 0 ? 0 : p];          // :227
        same += (pred_tokens[(size_t)b * L + a] == oracle) && align;  // :230
        // number-random and cmlm: the glance scores (:235-236, 245-246); default strategy: the alignment mask itself
        s_prob[a] = strategy == PCFGNAT_GLANCE_DEFAULT ? (align ? 1.f : 0.f) : (align ? noise[(size_t)b * L + a] : -100.f);
    }
    same = (int)wave_sum((float)same);
    if ((tid & 63) == 0) atomicAdd(&s_same, same);
    __syncthreads();
    const int total_same = s_same;
    // glance_nums = ((target_length - same_num) * context_p + 0.5).to(long) in float32 (:237); cmlm: a uniform fraction of
    // the target length instead (:247); the default strategy has none
    const int64_t glance = strategy == PCFGNAT_GLANCE_CMLM      ? (int64_t)((float)n * length_rand[b] + 0.5f)
                           : strategy == PCFGNAT_GLANCE_DEFAULT ? 0
                                                                : (int64_t)((float)(n - total_same) * context_p + 0.5f);
    if (tid == 0) {
        same_num[b] = total_same;
        glance_nums[b] = glance;
    }
    // match mask [T][L]: node a carries target position t (:225)
    unsigned char *mm = matchmask + (size_t)b * T * L;
    for (int i = tid; i < T * L; i += GNT) {
        const int t = i / L, a = i - t * L;
        mm[i] = s_path[a] == t;
    }
    // threshold = the glance-th largest noise value (:238-240); every thread ranks its own values
    if (glance != 0 && strategy != PCFGNAT_GLANCE_DEFAULT) {
        const int64_t k = (glance - 1 < 0) ? 0 : (glance - 1 >= L ? L - 1 : glance - 1);  // index into the descending order
        for (int a = tid; a < L; a += GNT) {
            const float v = s_prob[a];
            int gt = 0, ge = 0;
            for (int o = 0; o < L; o++) {
                const float w = s_prob[o];
                gt += w > v;
                ge += w >= v;
            }
            if (gt <= k && k < ge) s_thresh = v;  // all writers hold the same value
        }
    }
    __syncthreads();
    const float thresh = s_thresh;
    // default strategy (:231-233): every aligned node is revealed with probability (n - same) / n * context_p, in float32
    const float share = (float)(n - total_same) / (float)n * context_p;
    for (int a = tid; a < L; a += GNT) {
        // number-random, cmlm: keep_prob is 0 or 1 and the uniform draw lies in [0, 1): rand < keep_prob is keep_prob
        // itself (:241, 253)
        const bool keep = strategy == PCFGNAT_GLANCE_DEFAULT ? keep_rand[(size_t)b * L + a] < share * s_prob[a] : s_prob[a] >= thresh;
        const int p = s_path[a];
        keep_mask[(size_t)b * L + a] = keep;
        glat_tokens[(size_t)b * L + a] = keep ? tg[p < 0 ? 0 : p] : prev_tokens[(size_t)b * L + a];  // :255
    }
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

extern "C" int pcfgnat_glat_step(const void *logits, int dtype, const int64_t *targets, const int64_t *prev_output_tokens,
                                 const float *links, int glance_strategy, const float *noise, const float *length_rand,
                                 const float *keep_rand, float context_p, int64_t pad_index, float *match_all,
                                 float *S, float *aux, int64_t *pred_tokens, int64_t *lengths, int64_t *path,
                                 unsigned char *matchmask, unsigned char *keep_word_mask, int64_t *glat_prev_output_tokens,
                                 int64_t *same_num, int64_t *glance_nums, float *loss_out, int64_t B, int64_t L, int64_t V,
                                 int64_t T, int64_t ml, void *stream) {
    PCFGNAT_REQUIRE(B >= 1 && L >= 4 && T >= 2 && V >= 1 && ml >= 0, "glat_step: bad dimensions");
    PCFGNAT_REQUIRE(L <= 4096 && T <= 4096, "glat_step: dimension too large (L, T <= 4096)");
    PCFGNAT_REQUIRE(logits && targets && prev_output_tokens && links && match_all && S && aux && pred_tokens && lengths &&
                        path && matchmask && keep_word_mask && glat_prev_output_tokens && same_num && glance_nums && loss_out,
                    "glat_step: null pointer");
    PCFGNAT_REQUIRE(glance_strategy == PCFGNAT_GLANCE_NUMBER_RANDOM || glance_strategy == PCFGNAT_GLANCE_CMLM ||
                        glance_strategy == PCFGNAT_GLANCE_DEFAULT,
                    "glat_step: unknown glance strategy %d", glance_strategy);
    PCFGNAT_REQUIRE(glance_strategy == PCFGNAT_GLANCE_DEFAULT ? keep_rand != nullptr : noise != nullptr,
                    "glat_step: the strategy's random numbers are missing (noise for number-random and cmlm, keep_rand for the default)");
    PCFGNAT_REQUIRE(glance_strategy != PCFGNAT_GLANCE_CMLM || length_rand != nullptr, "glat_step: cmlm needs length_rand");
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(glat_lengths_kernel, dim3((unsigned)B), dim3(GNT), 0, s, prev_output_tokens, targets, pad_index, lengths, (int)B,
                       (int)L, (int)T);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    const int64_t *ol = lengths, *tl = lengths + B;
    int rc = lsg_forward_eos_argmax(logits, dtype, targets, match_all, pred_tokens, ol, tl, B, L, V, T, stream);
    if (rc != PCFGNAT_OK) return rc;
    rc = pcfgnat_pcfg_loss(match_all, links, ol, tl, S, aux, B, L, T, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    rc = pcfgnat_pcfg_best_tree(S, aux, match_all, links, ol, tl, path, B, L, T, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    const int64_t Mc = (L - 2) / (ml + 1) + 1;
    const size_t dyn = (size_t)2 * L * sizeof(float);
    hipLaunchKernelGGL(glat_glue_kernel, dim3((unsigned)B), dim3(GNT), dyn, s, path, targets, prev_output_tokens, pred_tokens, noise,
                       length_rand, keep_rand, glance_strategy, lengths, context_p, matchmask, keep_word_mask, glat_prev_output_tokens, same_num, glance_nums, (int)B, (int)L, (int)T,
                       LossTask{S, tl, loss_out, (int)B, Mc * (T + 2)});
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
