// PCFG inside algorithm (loss forward), its exact backward, and the GLAT best-tree trace, for max_left = 1.
//
// Replaces the reference's pcfg_loss.cu (calculate_C_kernel :262-349, calculate_S_kernel :84-224),
// pcfg_loss_backward.cu (seven kernels, :28-603) and pcfg_best_tree.cu (:64-301).
//
// With max_left = 1 (every shipped configuration) main-chain node a = 2*a_id+1 has one local leaf a-1 and the
// recurrences collapse to
//   S[a][s] = LSE( match[a][s]                 + F0[a][s+1],      F0[a][t] = LSE_{c>=a} links[a][0][c] + S[c][t]
//                  match[a-1][s] + match[a][s+1] + F1[a][s+2] )     F1[a][t] = LSE_{c>=a} links[a][1][c] + S[c][t]
// and, with the outside score beta[c][t] = log(dS[root][0]/dS[c][t]) - ... (posterior = exp(beta + S)),
//   beta[c][t] = LSE_{a<=c}( links[a][0][c] + match[a][t-1] + beta[a][t-1],
//                            links[a][1][c] + match[a-1][t-2] + match[a][t-1] + beta[a][t-2] ).
//
// Design (latency-bound sweeps over the target positions, one workgroup of 512 threads per sentence and sweep): the
// sentence's compact link matrices live in registers for the whole sweep (one 8-lane group per node, lanes strided over
// the other index), the current column of S (or of the outside weights) is exchanged through LDS, one workgroup barrier
// per target position.  The forward leaves F0/F1 behind so that the backward needs a single outside sweep; that sweep
// reads links, emissions and its own earlier columns only, so in the single call the two run side by side as two
// workgroups (inside_pair_ml1_kernel) and a parallel kernel multiplies their tables into the posteriors
// (inside_combine_ml1_kernel); in the two-call API the outside sweep accumulates rule posteriors in registers and
// emission posteriors come from an element-wise epilogue.
// Graphs of more than 130 nodes use the streaming or the pipelined sweeps (link rows from L2, or spread over several
// workgroups per sentence).
//
// One translation unit, cut by kernel family: inside_common.hip.h (table layouts), inside_short.hip.h (graphs of up to 130
// nodes), inside_best_tree.hip.h, inside_stream.hip.h (one workgroup per long sentence), inside_pipe.hip.h (pipelines of
// workgroups per long sentence), inside_posteriors.hip.h (posteriors of long graphs); this file holds the launch logic and
// the C-ABI entry points.
#include "common.hip.h"
#include "glat_glue.hip.h"
#include "inside_common.hip.h"
#include "inside_short.hip.h"
#include "inside_best_tree.hip.h"
#include "inside_stream.hip.h"
#include "inside_pipe.hip.h"
#include "inside_posteriors.hip.h"

#include <atomic>
#include <mutex>

namespace pcfgnat {
namespace {

__global__ void fill_zero_kernel(float *p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.f;
}


// loss = -(1/B) * sum_b [ll_b finite] ll_b / n_b and the number of invalid sentences (nat_pcfg_loss.py:123-135), reduced
// in a fixed order by one workgroup.  out[0] = loss, out[1] = invalid count.
__global__ __launch_bounds__(256) void criterion_loss_kernel(const float *__restrict__ S, const int64_t *__restrict__ tgt_len,
                                                            float *__restrict__ out, int B, int Mc, int T, float *__restrict__ ll_out) {
    criterion_loss_block<256>(LossTask{S, tgt_len, out, B, (int64_t)Mc * (T + 2), ll_out});
}

// The pipelined sweeps are used while a batch needs no more than g_pipeline_max_wg workgroups.  The default is no limit in
// practice: measured at 512 graph nodes and 140 target tokens they beat one workgroup per sentence 3.5x at 16 sentences
// and still 1.8x at 512 sentences (8192 workgroups: the blocks of a sentence are adjacent in dispatch order, leading
// block first, so a block never waits for one that has not been started).  Both numbers can be changed through
// pcfgnat_pipeline_config.
std::atomic<int> g_pipeline_max_wg{1 << 20}, g_pipeline_spin_limit{PCFGNAT_DEFAULT_SPIN_LIMIT};
std::atomic<int> g_pipeline_spin_limit_outside{-1};  // side-by-side launch only; negative: the common limit
// Bound of the one wait of the second-chance launch (the outside sweep's workgroup for the forward's, where both are
// redone), in polls of about a microsecond.  pcfgnat_pipeline_redo_wait_limit.
constexpr int DEFAULT_REDO_WAIT_LIMIT = 1 << 23;
std::atomic<int> g_redo_wait_limit{DEFAULT_REDO_WAIT_LIMIT};
// Largest base-2 exponent a factor of the rule posteriors of long graphs may have on the matrix cores (see
// links_grad_ml1_stream_kernel); a tile beyond it is recomputed term by term.  pcfgnat_links_grad_range_limit.
std::atomic<float> g_links_grad_range_limit{120.f};
// How a call sweeps its long graphs, decided once per call from one reading of the process-wide setting (a setting that
// changes while a call is being enqueued must not reach half of its launches).
struct PipelinePlan {
    int NQ;             // chunks of 64 nodes per sentence; 0: the pipelined sweeps do not apply
    bool side_by_side;  // forward and outside pipeline in one launch
};
PipelinePlan pipeline_plan(int B, int T, int Mc) {
    const int max_wg = g_pipeline_max_wg.load();
    const int NQ = stream_mp(Mc) / 64, CL = 64 * NQ / NLP;
    PipelinePlan plan{0, false};
    if (NQ >= 2 && NQ <= 8 && T + 2 < 4096 && (int64_t)B * CL <= max_wg) {
        plan.NQ = NQ;
        plan.side_by_side = (int64_t)2 * B * CL <= max_wg;
    }
    return plan;
}

template <int NQ>
int launch_fwd_pipe(const float *match_all, const int64_t *ol, const int64_t *tl, float *S, float *aux, int B, int L, int T, int Mc,
                    hipStream_t stream, bool both) {
    constexpr int CL = 64 * NQ / NLP;
    const size_t match_bytes = (size_t)2 * NLP * T * sizeof(float);
    if (both) {  // the outside pipeline in the same launch, behind the forward one in dispatch order
        const int spin_out = g_pipeline_spin_limit_outside.load() >= 0 ? g_pipeline_spin_limit_outside.load() : g_pipeline_spin_limit.load();
        // while every block of both pipelines can have a compute unit of its own: claim more than half of a unit's LDS so
        // that no two blocks share one (and its instruction issue), and spread the outside sweep's collecting over four waves
        const bool roomy = 2 * B * CL <= device_compute_units();
        if (match_bytes <= LDS_BUDGET - 8192) {
            const size_t lds = (roomy && match_bytes < PAD_EXCLUSIVE_LDS) ? PAD_EXCLUSIVE_LDS : match_bytes;
            if (roomy) {
                auto k = inside_both_ml1_pipe_kernel<NQ, true, 4>;
                PCFGNAT_DYNAMIC_LDS(k, lds);
                hipLaunchKernelGGL(k, dim3(2 * B * CL), dim3(16 * NLP + 256), lds, stream, match_all, ol, tl, S, aux, L, T, Mc,
                                   g_pipeline_spin_limit.load(), spin_out, B * CL);
            } else {
                auto k = inside_both_ml1_pipe_kernel<NQ, true, 1>;
                PCFGNAT_DYNAMIC_LDS(k, lds);
                hipLaunchKernelGGL(k, dim3(2 * B * CL), dim3(NTP), lds, stream, match_all, ol, tl, S, aux, L, T, Mc,
                                   g_pipeline_spin_limit.load(), spin_out, B * CL);
            }
        } else {
            hipLaunchKernelGGL((inside_both_ml1_pipe_kernel<NQ, false, 1>), dim3(2 * B * CL), dim3(NTP), 0, stream, match_all, ol, tl, S, aux,
                               L, T, Mc, g_pipeline_spin_limit.load(), spin_out, B * CL);
        }
    } else if (match_bytes <= LDS_BUDGET - 8192 && B * CL <= device_compute_units()) {  // a compute unit per block: four collector waves
        auto k = inside_fwd_ml1_pipe_kernel<NQ, true, 4>;
        const size_t lds = match_bytes < PAD_EXCLUSIVE_LDS ? PAD_EXCLUSIVE_LDS : match_bytes;
        PCFGNAT_DYNAMIC_LDS(k, lds);
        hipLaunchKernelGGL(k, dim3(B * CL), dim3(16 * NLP + 256), lds, stream, match_all, ol, tl, S, aux, L, T, Mc,
                           g_pipeline_spin_limit.load());
    } else if (match_bytes <= LDS_BUDGET - 8192) {
        auto k = inside_fwd_ml1_pipe_kernel<NQ, true>;
        PCFGNAT_DYNAMIC_LDS(k, match_bytes);
        hipLaunchKernelGGL(k, dim3(B * CL), dim3(NTP), match_bytes, stream, match_all, ol, tl, S, aux, L, T, Mc,
                           g_pipeline_spin_limit.load());
    } else {
        hipLaunchKernelGGL((inside_fwd_ml1_pipe_kernel<NQ, false>), dim3(B * CL), dim3(NTP), 0, stream, match_all, ol, tl, S, aux, L, T,
                           Mc, g_pipeline_spin_limit.load());
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    if (both) return PCFGNAT_OK;  // rebased together with the outside tables, once the redo of the forward has run
    hipLaunchKernelGGL(pipeline_rebase_kernel, dim3(CL - 1, B), dim3(256), (size_t)(T + 2) * sizeof(double), stream, aux, ol, tl, L, T,
                       Mc);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
template <int NQ>
int launch_bwd_pipe(const float *S, float *aux, const float *match_all, const int64_t *ol, const int64_t *tl, int B, int L, int T,
                    int Mc, hipStream_t stream) {
    constexpr int CL = 64 * NQ / NLP;
    const size_t base = (size_t)(T + 4) * sizeof(float), with_match = base + (size_t)2 * NLP * T * sizeof(float);
    if (with_match <= LDS_BUDGET - 8192) {
        auto k = inside_bwd_ml1_pipe_kernel<NQ, true>;
        PCFGNAT_DYNAMIC_LDS(k, with_match);
        hipLaunchKernelGGL(k, dim3(B * CL), dim3(NTP), with_match, stream, S, aux, match_all, ol, tl, L, T, Mc,
                           g_pipeline_spin_limit.load());
    } else {
        hipLaunchKernelGGL((inside_bwd_ml1_pipe_kernel<NQ, false>), dim3(B * CL), dim3(NTP), base, stream, S, aux, match_all, ol, tl, L,
                           T, Mc, g_pipeline_spin_limit.load());
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// zero_slabs: links_grad, where the call also has the backward to do (its slab is then zeroed here, beside the compact copies)
int launch_fwd_stream(const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux, int B,
                      int L, int T, int Mc, hipStream_t stream, int NQ, bool side_by_side = false, float *zero_slabs = nullptr) {
    const int MP = stream_mp(Mc);
    PCFGNAT_REQUIRE(((uintptr_t)aux & 15) == 0, "pcfg_loss: aux must be 16-byte aligned");
    hipLaunchKernelGGL(compact_links_ml1_kernel, dim3(MP / 32, MP / 32, B), dim3(256), 0, stream, links, ol, aux, L, T, Mc, MP, zero_slabs);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    // pipelined sweep first where it applies; the one-workgroup sweep then only redoes sentences whose blocks gave up
    int rc = PCFGNAT_OK;
    switch (NQ) {
        case 2: rc = launch_fwd_pipe<2>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 3: rc = launch_fwd_pipe<3>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 4: rc = launch_fwd_pipe<4>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 5: rc = launch_fwd_pipe<5>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 6: rc = launch_fwd_pipe<6>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 7: rc = launch_fwd_pipe<7>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        case 8: rc = launch_fwd_pipe<8>(match_all, ol, tl, S, aux, B, L, T, Mc, stream, side_by_side); break;
        default: break;
    }
    if (rc != PCFGNAT_OK) return rc;
    const int only_flagged = NQ != 0;
    const size_t base = ((size_t)4 * MP + 32) * sizeof(float);
    const size_t with_match = base + (size_t)2 * Mc * T * sizeof(float);
    if (side_by_side) {
        // both pipelines have run: one launch for the second chance of either sweep (in the normal case it finds no flag
        // set and ends at once), then both sweeps' tables to common offsets and the corrections of the posteriors
        const size_t base_bwd = ((size_t)5 * MP + T + 4) * sizeof(float);
        const size_t lds = base > base_bwd ? base : base_bwd;
        const int WAIT_LIMIT = g_redo_wait_limit.load();  // polls of about a microsecond
        if (Mc <= NT / 4)
            hipLaunchKernelGGL(inside_redo_ml1_stream_kernel<4>, dim3(B, 2), dim3(NT), lds, stream, match_all, links, ol, tl, S, aux, L, T,
                               Mc, MP, WAIT_LIMIT);
        else
            hipLaunchKernelGGL(inside_redo_ml1_stream_kernel<8>, dim3(B, 2), dim3(NT), lds, stream, match_all, links, ol, tl, S, aux, L, T,
                               Mc, MP, WAIT_LIMIT);
        PCFGNAT_HIP_CHECK(hipGetLastError());
        const int CL = 64 * NQ / NLP;
        hipLaunchKernelGGL(pipeline_finish_kernel, dim3(2 * CL - 1, B), dim3(256), (size_t)2 * (T + 4) * sizeof(double), stream, aux, ol, tl,
                           L, T, Mc, CL, S);
        PCFGNAT_HIP_CHECK(hipGetLastError());
        return PCFGNAT_OK;
    }
    if (with_match <= LDS_BUDGET) {
        auto k = inside_fwd_ml1_stream_kernel<true, 4>;
        PCFGNAT_DYNAMIC_LDS(k, with_match);
        hipLaunchKernelGGL(k, dim3(B), dim3(NT), with_match, stream, match_all, links, ol, tl, S, aux, L, T, Mc, MP, only_flagged);
    } else {
        hipLaunchKernelGGL((inside_fwd_ml1_stream_kernel<false, 4>), dim3(B), dim3(NT), base, stream, match_all, links, ol, tl, S, aux, L,
                           T, Mc, MP, only_flagged);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// side_by_side: the outside pipeline has already run, beside the forward one (launch_both_stream): only the redo of the
// sentences it gave up and the posteriors (with their per-column corrections) are left to do.
int launch_bwd_stream(const float *go, const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol,
                      const int64_t *tl, float *mg, float *lg, int B, int L, int T, int Mc, Seed seed, hipStream_t stream, int NQ,
                      bool side_by_side = false, bool slabs_zeroed = false) {
    const int MP = stream_mp(Mc);
    const int tiles = (Mc + LG_TILE - 1) / LG_TILE;
    PCFGNAT_REQUIRE(((uintptr_t)aux & 15) == 0, "pcfg_loss_backward: aux must be 16-byte aligned");
    const size_t base = ((size_t)5 * MP + T + 4) * sizeof(float);
    const size_t with_match = base + (size_t)2 * Mc * T * sizeof(float);
    int rc = PCFGNAT_OK;
    switch (side_by_side ? 0 : NQ) {
        case 2: rc = launch_bwd_pipe<2>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 3: rc = launch_bwd_pipe<3>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 4: rc = launch_bwd_pipe<4>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 5: rc = launch_bwd_pipe<5>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 6: rc = launch_bwd_pipe<6>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 7: rc = launch_bwd_pipe<7>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        case 8: rc = launch_bwd_pipe<8>(S, aux, match_all, ol, tl, B, L, T, Mc, stream); break;
        default: break;
    }
    if (rc != PCFGNAT_OK) return rc;
    const int only_flagged = NQ != 0;
    // lanes per node: four while one pass covers all nodes; beyond that the outside sweep measured faster with eight
    if (side_by_side) {
        // (the outside sweep's second chance has run in the launch it shares with the forward's: launch_fwd_stream)
    } else if (with_match <= LDS_BUDGET) {
        auto k = Mc <= NT / 4 ? inside_bwd_ml1_stream_kernel<true, 4> : inside_bwd_ml1_stream_kernel<true, 8>;
        PCFGNAT_DYNAMIC_LDS(k, with_match);
        hipLaunchKernelGGL(k, dim3(B), dim3(NT), with_match, stream, S, aux, match_all, ol, tl, L, T, Mc, MP, only_flagged);
    } else {
        auto k = Mc <= NT / 4 ? inside_bwd_ml1_stream_kernel<false, 4> : inside_bwd_ml1_stream_kernel<false, 8>;
        hipLaunchKernelGGL(k, dim3(B), dim3(NT), base, stream, S, aux, match_all, ol, tl, L, T, Mc, MP, only_flagged);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    if (!slabs_zeroed) {
        const size_t nlg = (size_t)B * L * 2 * L;
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, stream, lg, nlg);
        PCFGNAT_HIP_CHECK(hipGetLastError());
    }
    const int use_corr = side_by_side ? 1 : 0;
    bool small;
    const int span = links_grad_span(T, (long)B * tiles * (tiles + 1) / 2, small);
    auto lgk = small ? links_grad_ml1_stream_kernel<LG_SPAN_SMALL / 32> : links_grad_ml1_stream_kernel<LG_SPAN / 32>;
    PCFGNAT_DYNAMIC_LDS(lgk, links_grad_lds_bytes(span));
    // The workgroups below the diagonal of the tile grid have no rules to do: they take the emission posteriors while that
    // leaves each of their threads a handful of cells; otherwise those get a launch of their own.
    const long spare_threads = (long)tiles * (tiles - 1) / 2 * 256;
    const bool emis_inside = spare_threads > 0 && (long)L * T <= 16 * spare_threads;
    hipLaunchKernelGGL(lgk, dim3(tiles, tiles, B), dim3(256), links_grad_lds_bytes(span), stream, go, S, aux, links, ol, tl, lg, L, T,
                       Mc, seed, use_corr, g_links_grad_range_limit.load(), span,
                       MatchGradArgs{match_all, emis_inside ? mg : nullptr});
    PCFGNAT_HIP_CHECK(hipGetLastError());
    if (!emis_inside) {
        hipLaunchKernelGGL(match_grad_ml1_stream_kernel, dim3((L * T + 255) / 256, B), dim3(256), 0, stream, go, S, aux, match_all, ol, tl,
                           mg, L, T, Mc, seed, use_corr);
        PCFGNAT_HIP_CHECK(hipGetLastError());
    }
    return PCFGNAT_OK;
}

template <int R>
int launch_fwd(const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux, int B, int L,
               int T, int Mc, hipStream_t stream) {
    const size_t base = ((size_t)head_floats(T) + 2 * 64 * R) * sizeof(float);
    const size_t with_tab = base + ((size_t)2 * Mc * T + (size_t)3 * Mc * (T + 2)) * sizeof(float);
    if (with_tab <= LDS_BUDGET) {
        auto k = inside_fwd_ml1_kernel<R, true>;
        PCFGNAT_DYNAMIC_LDS(k, with_tab);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), with_tab, stream, match_all, links, ol, tl, S, aux, L, T, Mc);
    } else {
        auto k = inside_fwd_ml1_kernel<R, false>;
        PCFGNAT_REQUIRE(base <= LDS_BUDGET, "pcfg_loss: target length %d too large for the column offsets in LDS", T);
        PCFGNAT_DYNAMIC_LDS(k, base);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), base, stream, match_all, links, ol, tl, S, aux, L, T, Mc);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

template <int R>
int launch_bwd(const float *go, const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol,
               const int64_t *tl, float *mg, float *lg, int B, int L, int T, int Mc, Seed seed, hipStream_t stream) {
    const size_t base = ((size_t)head_floats(T) + 4 * 64 * R) * sizeof(float);
    const size_t with_tab = base + ((size_t)2 * Mc * T + (size_t)4 * Mc * (T + 2)) * sizeof(float);
    if (with_tab <= LDS_BUDGET) {
        auto k = inside_bwd_ml1_kernel<R, true>;
        PCFGNAT_DYNAMIC_LDS(k, with_tab);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), with_tab, stream, go, S, aux, match_all, links, ol, tl, mg, lg, L, T, Mc, seed);
    } else {
        auto k = inside_bwd_ml1_kernel<R, false>;
        PCFGNAT_REQUIRE(base <= LDS_BUDGET, "pcfg_loss_backward: target length %d too large for the column offsets in LDS", T);
        PCFGNAT_DYNAMIC_LDS(k, base);
        hipLaunchKernelGGL(k, dim3(B), dim3(NTR), base, stream, go, S, aux, match_all, links, ol, tl, mg, lg, L, T, Mc, seed);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// Returns PCFGNAT_EUNSUPPORTED (without a message being an error for the caller) when the fused kernel does not apply.
template <int R>
int launch_fused(const float *go, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux,
                 float *mg, float *lg, int B, int L, int T, int Mc, Seed seed, hipStream_t stream, bool *done,
                 PadFill pad = PadFill{nullptr, 0}, bool *pad_done = nullptr, const LossTask *loss = nullptr, bool *loss_done = nullptr) {
    const size_t need = ((size_t)head_floats(T) + 4 * 64 * R + (size_t)4 * Mc * (T + 2) + (size_t)2 * Mc * T) * sizeof(float);
    *done = false;
    if (R == 1) {  // the two sweeps side by side as two workgroups per sentence, then the posteriors
        const size_t fwd_bytes = ((size_t)head_floats(T) + 2 * 64 + (size_t)2 * Mc * T + (size_t)3 * Mc * (T + 2)) * sizeof(float);
        const size_t pair_bytes = fwd_bytes > outside_role_bytes(Mc, T) ? fwd_bytes : outside_role_bytes(Mc, T);
        const size_t comb_bytes = ((size_t)(T + 4) + (size_t)Mc * (T + 2) + (size_t)8 * (T + 2)) * sizeof(float);
        if (pair_bytes <= LDS_BUDGET && comb_bytes <= 64 * 1024 && L <= 128) {
            PCFGNAT_REQUIRE(((uintptr_t)aux & 7) == 0, "pcfg_loss_forward_backward: aux must be 8-byte aligned");
            PCFGNAT_DYNAMIC_LDS(inside_pair_ml1_kernel, pair_bytes);
            // the fill rides along only while the sweeps leave compute units free for it (the gather backward writes the
            // zeros itself otherwise)
            const bool fill = pad.base != nullptr && pad.row_bytes > 0 && 2 * B <= pad_max_sweep_wgs();
            // With the fill, every workgroup of the launch claims more than half of a compute unit's LDS, so that no fill
            // workgroup shares a compute unit (and its instruction issue) with a sweep.
            const size_t launch_bytes = (fill && pair_bytes < PAD_EXCLUSIVE_LDS) ? PAD_EXCLUSIVE_LDS : pair_bytes;
            if (launch_bytes != pair_bytes)
                PCFGNAT_DYNAMIC_LDS(inside_pair_ml1_kernel, launch_bytes);
            hipLaunchKernelGGL(inside_pair_ml1_kernel, dim3((2 + (fill ? PAD_WGS : 0)) * B), dim3(NTR), launch_bytes, stream, match_all,
                               links, ol, tl, S, aux, L, T, Mc, B, pad);
            PCFGNAT_HIP_CHECK(hipGetLastError());
            if (fill && pad_done) *pad_done = true;
            const bool with_loss = loss != nullptr && loss->out != nullptr;
            hipLaunchKernelGGL(inside_combine_ml1_kernel, dim3(16, B + (with_loss ? 1 : 0)), dim3(256), comb_bytes, stream, go, S, aux,
                               match_all, links, ol, tl, mg, lg, L, T, Mc, seed,
                               with_loss ? *loss : LossTask{nullptr, nullptr, nullptr, 0, 0, nullptr});
            PCFGNAT_HIP_CHECK(hipGetLastError());
            if (with_loss && loss_done) *loss_done = true;
            *done = true;
            return PCFGNAT_OK;
        }
    }
    if (need > LDS_BUDGET) return PCFGNAT_OK;
    auto k = inside_fused_ml1_kernel<R>;
    PCFGNAT_DYNAMIC_LDS(k, need);
    hipLaunchKernelGGL(k, dim3(B), dim3(NTR), need, stream, go, match_all, links, ol, tl, S, mg, lg, L, T, Mc, seed);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    *done = true;
    return PCFGNAT_OK;
}

int check_dims(const char *who, int64_t B, int64_t L, int64_t T, int64_t ml) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 4 && T >= 2, "%s: need B >= 0, L >= 4, T >= 2 (got B=%lld L=%lld T=%lld)", who, (long long)B,
                    (long long)L, (long long)T);
    PCFGNAT_REQUIRE(ml >= 0, "%s: links must have at least one left option", who);
    PCFGNAT_REQUIRE(L <= 4096 && T <= 4096 && B <= 65535, "%s: dimension too large (L, T <= 4096, B <= 65535)", who);
    PCFGNAT_REQUIRE(ml <= 63 && L >= ml + 3, "%s: max_left = %lld needs a graph of at least max_left + 3 nodes (and max_left <= 63)", who,
                    (long long)ml);
    return PCFGNAT_OK;
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

int pcfgnat::pipeline_max_workgroups() { return g_pipeline_max_wg.load(); }
int pcfgnat::pipeline_spin_limit() { return g_pipeline_spin_limit.load(); }

extern "C" void pcfgnat_pipeline_config(int max_workgroups, int spin_limit) {
    if (max_workgroups >= 0) g_pipeline_max_wg.store(max_workgroups);
    if (spin_limit >= 0) g_pipeline_spin_limit.store(spin_limit);
}

extern "C" void pcfgnat_pipeline_outside_spin_limit(int spin_limit) { g_pipeline_spin_limit_outside.store(spin_limit); }

extern "C" void pcfgnat_links_grad_range_limit(float log2_limit) { g_links_grad_range_limit.store(log2_limit); }

extern "C" void pcfgnat_pipeline_redo_wait_limit(int polls) { g_redo_wait_limit.store(polls < 0 ? DEFAULT_REDO_WAIT_LIMIT : polls); }

extern "C" int pcfgnat_pipeline_redo_counts(unsigned long long *inside_sweeps, unsigned long long *viterbi_sentences,
                                            unsigned long long *inside_given_up, int reset) {
    PCFGNAT_REQUIRE(inside_sweeps && viterbi_sentences && inside_given_up, "pipeline_redo_counts: null pointer");
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(inside_sweeps, HIP_SYMBOL(g_inside_redone), sizeof(*inside_sweeps)));
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(inside_given_up, HIP_SYMBOL(g_inside_given_up), sizeof(*inside_given_up)));
    if (reset) {
        const unsigned long long zero = 0;
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_inside_redone), &zero, sizeof(zero)));
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_inside_given_up), &zero, sizeof(zero)));
    }
    return viterbi_redo_count(viterbi_sentences, reset);
}

extern "C" size_t pcfgnat_pcfg_aux_floats(int64_t B, int64_t L, int64_t T, int64_t ml) {
    if (B <= 0 || L < 2 || T < 0 || ml < 0) return 0;
    if (ml != 1) return generic_aux_floats(B, L, T, ml);
    const int64_t Mc = (L - 2) / (ml + 1) + 1;
    if (Mc <= 64) return (size_t)B * aux_stride_reg((int)Mc, (int)T);
    return (size_t)B * aux_stride_stream((int)Mc, (int)T);
}

extern "C" int pcfgnat_pcfg_loss(const float *match_all, const float *links, const int64_t *output_length,
                                 const int64_t *target_length, float *S, float *aux, int64_t B, int64_t L, int64_t T, int64_t ml,
                                 void *stream) {
    int rc = check_dims("pcfg_loss", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(match_all && links && output_length && target_length && S && aux, "pcfg_loss: null pointer");
    if (ml != 1) return generic_forward(match_all, links, output_length, target_length, S, aux, B, L, T, ml, stream);
    const int Mc = (int)((L - 2) / 2 + 1);
    hipStream_t s = (hipStream_t)stream;
    if (Mc <= 64) return launch_fwd<1>(match_all, links, output_length, target_length, S, aux, (int)B, (int)L, (int)T, Mc, s);
    return launch_fwd_stream(match_all, links, output_length, target_length, S, aux, (int)B, (int)L, (int)T, Mc, s,
                             pipeline_plan((int)B, (int)T, Mc).NQ);
}

int pcfgnat::inside_backward_impl(const float *grad_output, const float *S, float *aux, const float *match_all, const float *links,
                                  const int64_t *output_length, const int64_t *target_length, float *match_all_grad, float *links_grad,
                                  int64_t B, int64_t L, int64_t T, int64_t ml, Seed seed, void *stream) {
    int rc = check_dims("pcfg_loss_backward", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(S && aux && match_all && links && output_length && target_length && match_all_grad && links_grad,
                    "pcfg_loss_backward: null pointer");
    if (ml != 1)
        return generic_backward(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T,
                                ml, seed, stream);
    const int Mc = (int)((L - 2) / 2 + 1);
    hipStream_t s = (hipStream_t)stream;
    if (Mc <= 64)
        return launch_bwd<1>(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, (int)B,
                             (int)L, (int)T, Mc, seed, s);
    return launch_bwd_stream(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, (int)B,
                             (int)L, (int)T, Mc, seed, s, pipeline_plan((int)B, (int)T, Mc).NQ);
}

extern "C" int pcfgnat_pcfg_loss_backward(const float *grad_output, const float *S, float *aux, const float *match_all,
                                          const float *links, const int64_t *output_length, const int64_t *target_length,
                                          float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                          void *stream) {
    return inside_backward_impl(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T,
                                ml, seed_of(B), stream);
}

int pcfgnat::inside_forward_backward_impl(const float *grad_output, const float *match_all, const float *links,
                                          const int64_t *output_length, const int64_t *target_length, float *S, float *aux,
                                          float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                          Seed seed, void *stream, PadFill pad, bool *pad_done, const LossTask *loss,
                                          bool *loss_done) {
    if (pad_done) *pad_done = false;
    if (loss_done) *loss_done = false;
    int rc = check_dims("pcfg_loss_forward_backward", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(match_all && links && output_length && target_length && S && aux && match_all_grad && links_grad,
                    "pcfg_loss_forward_backward: null pointer");
    const int Mc = (int)((L - 2) / 2 + 1);
    hipStream_t s = (hipStream_t)stream;
    bool done = false;
    if (ml == 3 && inside_ml3_supported(L, T) && ((uintptr_t)links_grad % 16) == 0) {
        // max_left = 3: the sentences whose rules the model can produce in one launch, the others by the plain kernels
        rc = inside_ml3_forward_backward(grad_output, match_all, links, output_length, target_length, S, match_all_grad, links_grad, B, L,
                                         T, seed, stream);
        if (rc != PCFGNAT_OK) return rc;
        rc = generic_forward(match_all, links, output_length, target_length, S, aux, B, L, T, ml, stream, 1);
        if (rc != PCFGNAT_OK) return rc;
        return generic_backward(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T, ml,
                                seed, stream, 1);
    }
    if (ml != 1) {
        // general max_left: the two plain kernels
    } else if (Mc <= 64)
        rc = launch_fused<1>(grad_output, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad, (int)B, (int)L,
                             (int)T, Mc, seed, s, &done, pad, pad_done, loss, loss_done);
    if (rc != PCFGNAT_OK || done) return rc;
    const PipelinePlan plan = (ml == 1 && Mc > 64) ? pipeline_plan((int)B, (int)T, Mc) : PipelinePlan{0, false};
    if (plan.side_by_side) {  // the two pipelined sweeps in one launch
        rc = launch_fwd_stream(match_all, links, output_length, target_length, S, aux, (int)B, (int)L, (int)T, Mc, s, plan.NQ, true,
                               links_grad);
        if (rc != PCFGNAT_OK) return rc;
        return launch_bwd_stream(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, (int)B,
                                 (int)L, (int)T, Mc, seed, s, plan.NQ, true, true);
    }
    rc = pcfgnat_pcfg_loss(match_all, links, output_length, target_length, S, aux, B, L, T, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    return inside_backward_impl(grad_output, S, aux, match_all, links, output_length, target_length, match_all_grad, links_grad, B, L, T,
                                ml, seed, stream);
}

extern "C" int pcfgnat_pcfg_loss_forward_backward(const float *grad_output, const float *match_all, const float *links,
                                                 const int64_t *output_length, const int64_t *target_length, float *S, float *aux,
                                                 float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T,
                                                 int64_t ml, void *stream) {
    return inside_forward_backward_impl(grad_output, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad,
                                        B, L, T, ml, seed_of(B), stream);
}

// ---------------------------------------------------------------------------------------------------------------
// pcfgnat_pcfg_loss_forward_backward for callers that cannot allocate device memory (code under HIP graph capture,
// serving loops, harnesses that forbid hipMalloc): the auxiliary table lives in a device array of fixed size that
// belongs to the library.  Every device the code object is loaded on holds its own copy of the array at its own
// address, looked up once per device; in host code the array's name is only a handle for that lookup, never an address.
// ---------------------------------------------------------------------------------------------------------------
namespace {
static __device__ __align__(256) float static_aux[PCFGNAT_STATIC_AUX_FLOATS];
constexpr int STATIC_AUX_MAX_DEVICES = 64;
float *g_static_aux_ptr[STATIC_AUX_MAX_DEVICES];
std::mutex g_static_aux_mutex;

// The address of the current device's copy of static_aux (looked up with that device current, kept for later calls).
int static_aux_address(float **out) {
    int dev = -1;
    PCFGNAT_HIP_CHECK(hipGetDevice(&dev));
    PCFGNAT_REQUIRE(dev >= 0 && dev < STATIC_AUX_MAX_DEVICES, "pcfg_loss_forward_backward_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_aux_mutex);
    if (g_static_aux_ptr[dev] == nullptr) {
        float *ptr = nullptr;
        PCFGNAT_HIP_CHECK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(static_aux)));
        if (ptr == nullptr) return pcfgnat::fail(PCFGNAT_EHIP, "pcfg_loss_forward_backward_static: no device address for the static table");
        g_static_aux_ptr[dev] = ptr;
    }
    *out = g_static_aux_ptr[dev];
    return PCFGNAT_OK;
}
}  // namespace

extern "C" size_t pcfgnat_static_aux_floats(void) { return (size_t)PCFGNAT_STATIC_AUX_FLOATS; }

extern "C" int pcfgnat_pcfg_loss_forward_backward_static(const float *grad_output, const float *match_all, const float *links,
                                                        const int64_t *output_length, const int64_t *target_length, float *S,
                                                        float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T,
                                                        int64_t ml, void *stream) {
    int rc = check_dims("pcfg_loss_forward_backward_static", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    const size_t need = pcfgnat_pcfg_aux_floats(B, L, T, ml);
    PCFGNAT_REQUIRE(need <= (size_t)PCFGNAT_STATIC_AUX_FLOATS,
                    "pcfg_loss_forward_backward_static: B=%lld L=%lld T=%lld max_left=%lld needs %zu floats of auxiliary table, the "
                    "library's static table holds %zu (use pcfgnat_pcfg_loss_forward_backward with a buffer of the caller's)",
                    (long long)B, (long long)L, (long long)T, (long long)ml, need, (size_t)PCFGNAT_STATIC_AUX_FLOATS);
    float *aux = nullptr;
    rc = static_aux_address(&aux);
    if (rc != PCFGNAT_OK) return rc;
    // every table the kernels read from aux is written earlier in the same call (arrival marks of the pipelined sweeps
    // included), so what an earlier call left in the array does not matter
    return inside_forward_backward_impl(grad_output, match_all, links, output_length, target_length, S, aux, match_all_grad, links_grad,
                                        B, L, T, ml, seed_of(B), stream);
}

int pcfgnat::criterion_loss_impl(const float *S, const int64_t *target_length, float *out, float *ll_out, int64_t B, int64_t L, int64_t T,
                                 int64_t ml, void *stream) {
    int rc = check_dims("criterion_loss", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    PCFGNAT_REQUIRE(B >= 1 && S && target_length && out, "criterion_loss: null pointer or empty batch");
    const int Mc = (int)((L - 2) / (ml + 1) + 1);
    hipLaunchKernelGGL(criterion_loss_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, S, target_length, out, (int)B, Mc, (int)T, ll_out);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_criterion_loss(const float *S, const int64_t *target_length, float *out, int64_t B, int64_t L, int64_t T,
                                      int64_t ml, void *stream) {
    return criterion_loss_impl(S, target_length, out, nullptr, B, L, T, ml, stream);
}

namespace pcfgnat {
// Best tree and the GLAT glue behind it in one launch (max_left = 1); glue.path receives the tree.
int best_tree_glue_ml1(const float *S, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, int64_t B,
                       int64_t L, int64_t T, const GlatGlueArgs &glue, void *stream) {
    const int Mc = (int)((L - 2) / 2 + 1);
    const size_t glue_bytes = ((size_t)3 * L + 2) * sizeof(float) + (size_t)T * sizeof(int64_t);
    size_t tables = (size_t)Mc * (T + 2) + (size_t)2 * Mc * T, with_links = tables + (size_t)2 * Mc * Mc;  // floats, rounded up to even
    tables += tables & 1;
    with_links += with_links & 1;
    PCFGNAT_REQUIRE(glue_bytes <= LDS_BUDGET, "glat_step: graph of %lld nodes too long", (long long)L);
#define PCFGNAT_TREE_GLUE(mode, floats)                                                                                               \
    do {                                                                                                                             \
        auto k = best_tree_glue_ml1_kernel<mode>;                                                                                    \
        const size_t lds = (size_t)(floats) * sizeof(float) + glue_bytes;                                                            \
        PCFGNAT_DYNAMIC_LDS(k, lds);                                                                                                 \
        hipLaunchKernelGGL(k, dim3((unsigned)B), dim3(BT_NT), lds, (hipStream_t)stream, S, match_all, links, ol, tl, (int)L, (int)T, Mc, \
                           (int)(floats), glue);                                                                                     \
    } while (0)
    if (with_links * sizeof(float) + glue_bytes <= LDS_BUDGET) PCFGNAT_TREE_GLUE(2, with_links);
    else if (tables * sizeof(float) + glue_bytes <= LDS_BUDGET) PCFGNAT_TREE_GLUE(1, tables);
    else PCFGNAT_TREE_GLUE(0, 0);
#undef PCFGNAT_TREE_GLUE
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
}  // namespace pcfgnat

extern "C" int pcfgnat_pcfg_best_tree(const float *S, float *aux, const float *match_all, const float *links,
                                      const int64_t *output_length, const int64_t *target_length, int64_t *tree, int64_t B, int64_t L,
                                      int64_t T, int64_t ml, void *stream) {
    int rc = check_dims("pcfg_best_tree", B, L, T, ml);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(S && match_all && links && output_length && target_length && tree, "pcfg_best_tree: null pointer");
    if (ml != 1) {
        PCFGNAT_REQUIRE(aux != nullptr, "pcfg_best_tree: the auxiliary table of pcfg_loss is required for max_left != 1");
        return generic_best_tree(S, aux, match_all, links, output_length, target_length, tree, B, L, T, ml, stream);
    }
    const int Mc = (int)((L - 2) / 2 + 1);
    const size_t tables = ((size_t)Mc * (T + 2) + (size_t)2 * Mc * T) * sizeof(float);
    const size_t with_links = tables + (size_t)2 * Mc * Mc * sizeof(float);
    if (with_links <= LDS_BUDGET) {
        auto k = best_tree_ml1_kernel<2>;
        PCFGNAT_DYNAMIC_LDS(k, with_links);
        hipLaunchKernelGGL(k, dim3((unsigned)B), dim3(BT_NT), with_links, (hipStream_t)stream, S, match_all, links, output_length,
                           target_length, tree, (int)L, (int)T, Mc);
    } else if (tables <= LDS_BUDGET) {
        auto k = best_tree_ml1_kernel<1>;
        PCFGNAT_DYNAMIC_LDS(k, tables);
        hipLaunchKernelGGL(k, dim3((unsigned)B), dim3(BT_NT), tables, (hipStream_t)stream, S, match_all, links, output_length,
                           target_length, tree, (int)L, (int)T, Mc);
    } else {
        hipLaunchKernelGGL(best_tree_ml1_kernel<0>, dim3((unsigned)B), dim3(BT_NT), 0, (hipStream_t)stream, S, match_all, links,
                           output_length, target_length, tree, (int)L, (int)T, Mc);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
