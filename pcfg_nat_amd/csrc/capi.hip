// Library-wide pieces of the C-ABI: version and the thread-local error message.
#include "common.hip.h"

#include <mutex>
#include <unordered_map>

namespace pcfgnat {
char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace pcfgnat

namespace pcfgnat {
namespace {
constexpr int MAX_DEVICES_SEEN = 64;
std::mutex g_device_facts_mutex;
int g_compute_units[MAX_DEVICES_SEEN] = {0};
std::unordered_map<const void *, size_t> g_dynamic_lds[MAX_DEVICES_SEEN];
}  // namespace

int device_compute_units() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES_SEEN) return 256;
    std::lock_guard<std::mutex> lock(g_device_facts_mutex);
    if (g_compute_units[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        g_compute_units[dev] = n;
    }
    return g_compute_units[dev];
}

int ensure_dynamic_lds(const void *kernel, size_t bytes) {
    int dev = 0;
    PCFGNAT_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES_SEEN) {  // beyond the table: set it every time
        PCFGNAT_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
        return PCFGNAT_OK;
    }
    std::lock_guard<std::mutex> lock(g_device_facts_mutex);
    size_t &have = g_dynamic_lds[dev][kernel];
    if (bytes > have) {
        PCFGNAT_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
        have = bytes;
    }
    return PCFGNAT_OK;
}
}  // namespace pcfgnat

extern "C" int pcfgnat_abi_version(void) { return 5; }

extern "C" const char *pcfgnat_last_error(void) { return pcfgnat::error_buffer(); }

// ---------------------------------------------------------------------------------------------------------------
// One call for the whole training pass of the criterion (fs_plugins/criterions/nat_pcfg_loss.py:98-145 and the backward
// autograd derives from it): gather with eos mask -> inside forward+backward seeded with -1/(n_b*B) -> in-place gather
// backward -> loss.  Nothing is allocated, everything is enqueued on the caller's stream.
// ---------------------------------------------------------------------------------------------------------------
extern "C" int pcfgnat_criterion_step(void *logits, int dtype, const int64_t *targets, const float *links,
                                      const int64_t *output_length, const int64_t *target_length, const unsigned char *matchmask,
                                      const unsigned char *keep_word_mask, float *match_all, float *S,
                                      float *aux, float *match_all_grad, float *links_grad, float *row_lse, float *loss_out, int64_t B,
                                      int64_t L, int64_t V, int64_t T, int64_t ml, float loss_scale,
                                      const float *loss_scale_dev, void *stream, void *const *events) {
    if (dtype != PCFGNAT_F16 && dtype != PCFGNAT_F32)
        return pcfgnat::fail(PCFGNAT_EUNSUPPORTED, "criterion_step: logits must be float16 or float32 (the PCFG kernels are float32)");
    PCFGNAT_REQUIRE(B >= 1 && L >= 4 && T >= 2 && V >= 1 && ml >= 0, "criterion_step: bad dimensions");
    PCFGNAT_REQUIRE(logits && targets && links && output_length && target_length && match_all && S && aux && match_all_grad &&
                        links_grad && row_lse && loss_out,
                    "criterion_step: null pointer");
    PCFGNAT_REQUIRE((matchmask == nullptr) == (keep_word_mask == nullptr),
                    "criterion_step: matchmask and keep_word_mask must be given together (or both be null)");
    hipStream_t s = (hipStream_t)stream;
    const size_t esz = (dtype == PCFGNAT_F16) ? 2 : 4;
    const int64_t Mc = (L - 2) / (ml + 1) + 1;
#define PCFGNAT_MARK(k)                                                                     \
    do {                                                                                    \
        if (events && events[k]) PCFGNAT_HIP_CHECK(hipEventRecord((hipEvent_t)events[k], s)); \
    } while (0)
    PCFGNAT_MARK(0);
    int rc = pcfgnat::lsg_forward_lse_force(logits, dtype, targets, match_all, row_lse, output_length, target_length, matchmask,
                                            keep_word_mask, B, L, V, T, s);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_MARK(1);
    PCFGNAT_MARK(2);
    // the rows of pad nodes of the logits gradient are zeroed beside the sweeps where the inside launch can host that
    bool pad_done = false;
    rc = pcfgnat::inside_forward_backward_impl(nullptr, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad,
                                               B, L, T, ml, pcfgnat::seed_of(B, loss_scale, loss_scale_dev), s,
                                               pcfgnat::PadFill{(unsigned char *)logits, (int64_t)V * (int64_t)esz}, &pad_done);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_MARK(3);
    PCFGNAT_MARK(4);
    // the loss is reduced by the first workgroup of the same launch (S is complete by now)
    rc = pcfgnat::lsg_backward_lse_with_loss(logits, dtype, targets, T, 0, 1, match_all_grad, row_lse, B, L, V, T, S, Mc * (T + 2),
                                             target_length, loss_out, keep_word_mask, output_length, pad_done ? 1 : 0, nullptr, s);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_MARK(5);
#undef PCFGNAT_MARK
    return PCFGNAT_OK;
}

// ---------------------------------------------------------------------------------------------------------------
// The same pass cut at the point where autograd cuts it: everything that does not depend on the loss's upstream gradient
// in the forward (gather, both sweeps, the emission and rule posteriors with the criterion's weights, the loss), the one
// pass that turns the logits into their gradient in the backward, where the upstream gradient - a scalar in device
// memory - multiplies the emission posteriors in float32 ahead of the single rounding to the logits' dtype (the
// reference scales its saved gradients before the cast as well: pcfg_loss.py:77-83, 176-177).  No host read anywhere.
// ---------------------------------------------------------------------------------------------------------------
extern "C" int pcfgnat_criterion_forward(void *logits, int dtype, const int64_t *targets, const float *links,
                                         const int64_t *output_length, const int64_t *target_length, const unsigned char *matchmask,
                                         const unsigned char *keep_word_mask, float *match_all, float *S, float *aux,
                                         float *match_all_grad, float *links_grad, float *row_lse, float *loss_out, float *ll_out,
                                         int *pad_rows_zeroed, int64_t B, int64_t L, int64_t V, int64_t T, int64_t ml, void *stream) {
    if (dtype != PCFGNAT_F16 && dtype != PCFGNAT_F32)
        return pcfgnat::fail(PCFGNAT_EUNSUPPORTED, "criterion_forward: logits must be float16 or float32 (the PCFG kernels are float32)");
    PCFGNAT_REQUIRE(B >= 1 && L >= 4 && T >= 2 && V >= 1 && ml >= 0, "criterion_forward: bad dimensions");
    PCFGNAT_REQUIRE(logits && targets && links && output_length && target_length && match_all && S && aux && match_all_grad &&
                        links_grad && row_lse && loss_out && pad_rows_zeroed,
                    "criterion_forward: null pointer");
    PCFGNAT_REQUIRE((matchmask == nullptr) == (keep_word_mask == nullptr),
                    "criterion_forward: matchmask and keep_word_mask must be given together (or both be null)");
    const size_t esz = (dtype == PCFGNAT_F16) ? 2 : 4;
    *pad_rows_zeroed = 0;
    int rc = pcfgnat::lsg_forward_lse_force(logits, dtype, targets, match_all, row_lse, output_length, target_length, matchmask,
                                            keep_word_mask, B, L, V, T, stream);
    if (rc != PCFGNAT_OK) return rc;
    bool pad_done = false, loss_done = false;
    // the loss is formed beside the posteriors where the kernels of this shape offer that, by a launch of its own otherwise
    const pcfgnat::LossTask loss{S, target_length, loss_out, (int)B, (int64_t)((L - 2) / (ml + 1) + 1) * (T + 2), ll_out};
    rc = pcfgnat::inside_forward_backward_impl(nullptr, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad,
                                               B, L, T, ml, pcfgnat::seed_of(B), stream,
                                               pcfgnat::PadFill{(unsigned char *)logits, (int64_t)V * (int64_t)esz}, &pad_done, &loss,
                                               &loss_done);
    if (rc != PCFGNAT_OK) return rc;
    *pad_rows_zeroed = pad_done ? 1 : 0;
    if (loss_done) return PCFGNAT_OK;
    return pcfgnat::criterion_loss_impl(S, target_length, loss_out, ll_out, B, L, T, ml, stream);
}

extern "C" int pcfgnat_criterion_backward(void *logits_inout, int dtype, const int64_t *targets, const float *match_all_grad,
                                          const float *row_lse, const unsigned char *keep_word_mask, const int64_t *output_length,
                                          int pad_rows_zeroed, const float *upstream_dev, float *links_grad_inout, int64_t B, int64_t L,
                                          int64_t V, int64_t T, int64_t ml, void *stream) {
    if (dtype != PCFGNAT_F16 && dtype != PCFGNAT_F32)
        return pcfgnat::fail(PCFGNAT_EUNSUPPORTED, "criterion_backward: logits must be float16 or float32");
    PCFGNAT_REQUIRE(B >= 1 && L >= 4 && T >= 2 && V >= 1 && ml >= 0, "criterion_backward: bad dimensions");
    PCFGNAT_REQUIRE(logits_inout && targets && match_all_grad && row_lse && output_length, "criterion_backward: null pointer");
    // the rule gradients take the same factor: one float per thread of the same launch
    const pcfgnat::ScaleTask rules{(links_grad_inout != nullptr && upstream_dev != nullptr) ? links_grad_inout : nullptr,
                                   (size_t)B * L * (ml + 1) * L};
    return pcfgnat::lsg_backward_lse_with_loss(logits_inout, dtype, targets, T, 0, 1, match_all_grad, row_lse, B, L, V, T, nullptr, 0,
                                               nullptr, nullptr, keep_word_mask, output_length, pad_rows_zeroed ? 1 : 0, upstream_dev,
                                               stream, rules);
}

// ---------------------------------------------------------------------------------------------------------------
// The decode as the model runs it (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416, 483-502): front-end and
// Viterbi decode enqueued by one call.
// ---------------------------------------------------------------------------------------------------------------
extern "C" int pcfgnat_viterbi_decode_logits(const void *logits, int dtype, int64_t V, float *best_lprob, int64_t *best_idx,
                                             const float *links, const int64_t *output_length, const int64_t *left_tree_mask,
                                             int64_t mask_dim, int64_t pad_index, const float *length_penalty, void *workspace,
                                             int64_t *out_tokens, float *out_tokens_f32, int64_t *out_count, int64_t *pred_length,
                                             int64_t B, int64_t L, int64_t ml, void *stream) {
    if (dtype != PCFGNAT_F16 && dtype != PCFGNAT_F32)
        return pcfgnat::fail(PCFGNAT_EUNSUPPORTED, "viterbi_decode_logits: logits must be float16 or float32 (the Viterbi tables are float32)");
    int rc = pcfgnat_logsoftmax_max(logits, dtype, best_lprob, best_idx, B, L, V, stream);
    if (rc != PCFGNAT_OK) return rc;
    return pcfgnat_viterbi_decode(best_lprob, links, output_length, best_idx, left_tree_mask, mask_dim, pad_index, length_penalty,
                                  workspace, out_tokens, out_tokens_f32, out_count, pred_length, B, L, ml, stream);
}
