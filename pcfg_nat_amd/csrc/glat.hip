// GLAT glancing (reference fs_plugins/criterions/nat_pcfg_loss.py:193-269, all three glance strategies: :231-233 the
// default, :235-242 `number-random`, :244-251 `cmlm`) as one native
// call: sentence lengths from the pad counts, fused log-softmax + gather + eos mask + arg max in one read of the logits,
// inside forward, best-tree alignment, and one small kernel per sentence for everything the criterion does with the
// alignment (path clipping, match mask, oracle tokens, number of correct predictions, glance threshold, revealed
// tokens).  The random numbers of the sampling step are drawn by the caller with its own generator, in the reference's
// order, so that the random stream is the one the torch code consumes.
#include "common.hip.h"
#include "glat_glue.hip.h"

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

// One workgroup per sentence: the glue as a kernel of its own (max_left != 1; with max_left = 1 the kernel that walks the
// tree runs it).  Dynamic LDS: 2 L floats.
__global__ __launch_bounds__(GNT) void glat_glue_kernel(GlatGlueArgs g) {
    extern __shared__ float dyn[];
    glat_glue_block<GNT>((int)blockIdx.x, g, dyn);
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
    const int64_t Mc = (L - 2) / (ml + 1) + 1;
    const GlatGlueArgs glue{path, targets, prev_output_tokens, pred_tokens, noise, length_rand, keep_rand, glance_strategy, lengths, context_p,
                            matchmask, keep_word_mask, glat_prev_output_tokens, same_num, glance_nums, (int)B, (int)L, (int)T,
                            LossTask{S, tl, loss_out, (int)B, Mc * (T + 2)}};
    if (ml == 1) return best_tree_glue_ml1(S, match_all, links, ol, tl, B, L, T, glue, stream);  // one launch for both
    rc = pcfgnat_pcfg_best_tree(S, aux, match_all, links, ol, tl, path, B, L, T, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    hipLaunchKernelGGL(glat_glue_kernel, dim3((unsigned)B), dim3(GNT), (size_t)2 * L * sizeof(float), s, glue);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
