// Library-wide pieces of the C-ABI: version and the thread-local error message.
#include "common.hip.h"

namespace pcfgnat {
char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace pcfgnat

extern "C" int pcfgnat_abi_version(void) { return 1; }

extern "C" const char *pcfgnat_last_error(void) { return pcfgnat::error_buffer(); }

// One call for the whole training pass of the criterion (fs_plugins/criterions/nat_pcfg_loss.py:98-145 and the backward
// autograd derives from it): gather with eos mask -> inside forward -> inside backward seeded with -1/(n_b*B) ->
// in-place gather backward -> loss.  Five kernels enqueued back to back; nothing is allocated.
extern "C" int pcfgnat_criterion_step(void *logits, int dtype, const int64_t *targets, const float *links,
                                      const int64_t *output_length, const int64_t *target_length, float *match_all, float *S,
                                      float *aux, float *match_all_grad, float *links_grad, float *loss_out, int64_t B, int64_t L,
                                      int64_t V, int64_t T, int64_t ml, void *stream, void *const *events) {
    if (dtype == PCFGNAT_F64)
        return pcfgnat::fail(PCFGNAT_EUNSUPPORTED, "criterion_step: float64 logits gather to float64, the PCFG kernels are float32");
    hipStream_t s = (hipStream_t)stream;
#define PCFGNAT_MARK(i)                                                        \
    do {                                                                       \
        if (events && events[i]) PCFGNAT_HIP_CHECK(hipEventRecord((hipEvent_t)events[i], s)); \
    } while (0)
    PCFGNAT_MARK(0);
    int rc = pcfgnat_logsoftmax_gather_eos(logits, dtype, targets, T, 0, 1, match_all, 1, output_length, target_length, B, L, V, T, stream);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_MARK(1);
    PCFGNAT_MARK(2);
    PCFGNAT_MARK(3);  // forward and backward run as one launch where the tables fit in LDS: bracketed together by 4..5
    PCFGNAT_MARK(4);
    rc = pcfgnat_pcfg_loss_forward_backward(nullptr, match_all, links, output_length, target_length, S, aux, match_all_grad,
                                            links_grad, B, L, T, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_MARK(5);
    PCFGNAT_MARK(6);
    rc = pcfgnat_logsoftmax_gather_backward(logits, dtype, targets, T, 0, 1, match_all_grad, B, L, V, T, stream);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_MARK(7);
#undef PCFGNAT_MARK
    return pcfgnat_criterion_loss(S, target_length, loss_out, B, L, T, ml, stream);
}
