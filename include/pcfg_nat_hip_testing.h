/*
 * Test hooks, tuning settings and diagnostic counters of libpcfg_nat_hip.so.  None of them has a counterpart in the
 * reference and no call of include/pcfg_nat_hip.h needs them: they exist so that tests can send sentences down the fallback
 * paths (bounded waits that expire at once, range limits that fail everywhere) and so that a caller can see when a
 * fallback was taken.  All settings are process-wide atomics (every thread, stream and device) that take effect with the
 * next call; the counters live on the current device and reading them synchronises with it.
 */
#ifndef PCFG_NAT_HIP_TESTING_H
#define PCFG_NAT_HIP_TESTING_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * The long-graph paths (max_left = 1; inside sweeps for 130 <= L <= 1026, the Viterbi sweep of pcfgnat_viterbi_decode for
 * 194 <= L <= 514): a sentence is swept by one workgroup per block of 16 main-chain nodes, the blocks following each other
 * as a pipeline, as long as the batch needs no more than max_workgroups of them (B * 4 * ceil((L/2)/64) <= max_workgroups,
 * default 2^20), and by one workgroup per sentence otherwise.  pcfgnat_pcfg_loss_forward_backward runs the forward and the
 * outside pipeline of a sentence side by side in one launch while twice that number fits, one after the other otherwise.
 * A block that waits for the one ahead of it for more than spin_limit rounds of polling (default 2^15, some tens of
 * milliseconds; the blocks of a sentence normally follow each other at about 2 us) gives the sentence up, and the
 * one-workgroup sweep redoes it in the same call; results are the same either way up to fp32 rounding.
 * max_workgroups = 0 switches the pipeline off; a negative argument leaves that setting unchanged.
 *
 * Progress: the waits rely on the leading blocks of a sentence having the lower workgroup indices and on workgroups being
 * started in index order, so that a block never waits for one that has not been started while it occupies the slot that
 * block needs.  HIP does not promise that order; where it does not hold (or where another tenant keeps the leading block
 * from running) the bounded wait expires and the sentence is redone, which costs time, never correctness.
 */
void pcfgnat_pipeline_config(int max_workgroups, int spin_limit);

/* A wait limit of its own for the outside pipeline where the two pipelines of a sentence run side by side; negative (the
 * default) = the common limit.  Lets a test make one of the two sweeps give up and be redone while the other completes. */
void pcfgnat_pipeline_outside_spin_limit(int spin_limit);

/* The bound of the one wait inside the second-chance launch (where both sweeps of a sentence are redone, the outside
 * sweep's workgroup waits for the forward's, which is running or done and waits for nobody), in polls of about a
 * microsecond; default 2^23, negative restores it.  A sentence whose wait expires is given up: its log-likelihood becomes
 * NaN - an invalid sentence for the criterion, never a wrong gradient - and inside_given_up below counts it.  0 makes
 * every such wait expire at once (tests). */
void pcfgnat_pipeline_redo_wait_limit(int polls);

/* The rule posteriors of graphs beyond 130 nodes are summed over the target positions on the matrix cores, as products of
 * two factors per term; a 32x32 tile of (parent, child) pairs in which the product of the largest factors would exceed
 * 2^log2_limit (default 120) is recomputed with one exponential per term instead, which has no range limit.  A limit of
 * -inf sends every tile down the second path. */
void pcfgnat_links_grad_range_limit(float log2_limit);

/* Switches the one-launch kernel for max_left = 3 on (1, the default) or off (0: the plain kernels serve every sentence),
 * so that tests can hold the two against each other; a negative value changes nothing.  Returns the previous setting. */
int pcfgnat_max_left3_tuned(int on);

/* Diagnostic counters of that kernel on the current device since the library was loaded (or the last reset): sentences it
 * served, and sentences it left to the plain kernels because their links hold a rule of a composite local tree. */
int pcfgnat_max_left3_counts(unsigned long long *served, unsigned long long *left_to_plain, int reset);

/* The same two counters for the Viterbi tables at max_left = 3 (pcfgnat_pcfg_viterbi and the decode calls built on it),
 * whose one-launch kernel the same switch turns on and off. */
int pcfgnat_max_left3_viterbi_counts(unsigned long long *served, unsigned long long *left_to_plain, int reset);

/* Diagnostic counters since the library was loaded (or the last reset) on the current device: inside sweeps (forward and
 * outside counted apart) and single-call Viterbi decodes that the one-workgroup kernels redid because a pipelined sweep
 * gave up, and sentences given up for good (see pcfgnat_pipeline_redo_wait_limit).  reset != 0 clears them.  A caller that
 * sees the first two grow outside tests is paying the bounded wait on those calls; the third must stay zero. */
int pcfgnat_pipeline_redo_counts(unsigned long long *inside_sweeps, unsigned long long *viterbi_sentences,
                                 unsigned long long *inside_given_up, int reset);

#ifdef __cplusplus
}
#endif
#endif /* PCFG_NAT_HIP_TESTING_H */
