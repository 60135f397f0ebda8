// Shared host/device helpers of libpcfg_nat_hip (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/pcfg_nat_hip.h"
#include "../../include/pcfg_nat_hip_testing.h"

namespace pcfgnat {

// ---- error reporting ------------------------------------------------------------------------------------------
char *error_buffer();  // thread-local, 512 bytes (defined in capi.hip)

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

#define PCFGNAT_HIP_CHECK(expr)                                                                        \
    do {                                                                                               \
        hipError_t _e = (expr);                                                                        \
        if (_e != hipSuccess) return ::pcfgnat::fail(PCFGNAT_EHIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

#define PCFGNAT_REQUIRE(cond, ...)                                       \
    do {                                                                 \
        if (!(cond)) return ::pcfgnat::fail(PCFGNAT_EINVAL, __VA_ARGS__); \
    } while (0)

// ---- per-device facts and settings, looked up once (capi.hip) ---------------------------------------------------
// Compute units of the current device (hipDeviceAttributeMultiprocessorCount; 256 on MI355X, fewer on a partition).
int device_compute_units();
// Allows `kernel` to be launched with `bytes` of dynamic LDS on the current device.  The attribute is set once per
// (device, kernel) and raised only when a larger size comes along, not on every launch.
int ensure_dynamic_lds(const void *kernel, size_t bytes);
#define PCFGNAT_DYNAMIC_LDS(kernel, bytes)                                                   \
    do {                                                                                     \
        int _rc = ::pcfgnat::ensure_dynamic_lds((const void *)(kernel), (size_t)(bytes));     \
        if (_rc != PCFGNAT_OK) return _rc;                                                   \
    } while (0)

// ---- internal entry points shared between translation units ---------------------------------------------------
// The criterion's own weights, used when grad_output is null: d(-(ll/n).mean() * factor)/d ll_b = -factor/(n_b * norm_B)
// (nat_pcfg_loss.py:135, 139-140; pcfg_loss.py:77-83 for the upstream factor).  norm_B is passed apart from the batch size
// so that a batch can be processed in slices; the factor is a host value times an optional scalar in device memory (an
// fp16 loss scale that only the device knows), both 1 by default.
struct Seed {
    int norm_B;
    float scale;
    const float *scale_dev;
};
inline Seed seed_of(int64_t norm_B, float scale = 1.0f, const float *scale_dev = nullptr) {
    return Seed{(int)norm_B, scale, scale_dev};
}
__device__ __forceinline__ float seed_weight(const float *grad_out, int b, int n, const Seed &sd) {
    if (grad_out) return grad_out[b];
    float g = -1.0f / ((float)n * (float)sd.norm_B);
    if (sd.scale_dev) g *= *sd.scale_dev;
    return g * sd.scale;
}
__device__ __forceinline__ double seed_weight(const double *grad_out, int b, int n, const Seed &sd) {
    if (grad_out) return grad_out[b];
    double g = -1.0 / ((double)n * (double)sd.norm_B);
    if (sd.scale_dev) g *= (double)*sd.scale_dev;
    return g * (double)sd.scale;
}
// A buffer that the gather backward multiplies by its device-side upstream factor on the way (the rule gradients of the
// criterion's backward: one float per thread of the launch, instead of a launch of their own).  p null: nothing to do.
struct ScaleTask {
    float *p;
    size_t n;
};
// Like the public functions of the same name, with the weights above in place of the batch size.
int inside_backward_impl(const float *grad_output, const float *S, float *aux, const float *match_all, const float *links,
                         const int64_t *output_length, const int64_t *target_length, float *match_all_grad, float *links_grad, int64_t B,
                         int64_t L, int64_t T, int64_t ml, Seed seed, void *stream);
// A side task for the launch that holds the sweeps of short graphs, which leaves most of the chip and all of the memory
// bandwidth idle: zero the rows of the pad nodes (at or beyond a sentence's output length) of a [B,L,row_bytes] buffer -
// the criterion step's logits, whose gradient rows they are.  base null: nothing to do.  *pad_done (if given) tells
// whether the path taken carried the task out.
struct PadFill {
    unsigned char *base;
    int64_t row_bytes;
};
int inside_forward_backward_impl(const float *grad_output, const float *match_all, const float *links, const int64_t *output_length,
                                 const int64_t *target_length, float *S, float *aux, float *match_all_grad, float *links_grad,
                                 int64_t B, int64_t L, int64_t T, int64_t ml, Seed seed, void *stream,
                                 PadFill pad = PadFill{nullptr, 0}, bool *pad_done = nullptr, const struct LossTask *loss = nullptr,
                                 bool *loss_done = nullptr);

// Read-only logsoftmax_gather over the [B,T] targets with the eos mask, which also returns the first arg max of every row;
// the rows of nodes at or beyond a sentence's output length are left unread (zeros in selected and argmax)
int lsg_forward_eos_argmax(const void *logits, int dtype, const int64_t *targets, void *selected, int64_t *argmax,
                           const int64_t *output_length, const int64_t *target_length, int64_t B, int64_t L, int64_t V, int64_t T,
                           void *stream);

// pcfgnat_logsoftmax_gather_backward_lse whose first workgroup also reduces the criterion's loss when loss_out is given
// (lsg.hip); rows with keep[row] != 0 get a zero gradient; with pad_output_length, the rows of nodes at or beyond a
// sentence's output length (whose grad_selected rows the caller guarantees to be all zero) are zeroed without being read,
// or left alone when the caller has zeroed them already (pad_rows_zeroed); gscale_dev (may be null): one float in device
// memory that multiplies grad_selected on the fly
int lsg_backward_lse_with_loss(void *logits_inout, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl, int64_t st,
                               const void *grad_selected, const void *lse, int64_t B, int64_t L, int64_t V, int64_t T,
                               const float *S, int64_t ll_stride, const int64_t *target_length, float *loss_out,
                               const unsigned char *keep, const int64_t *pad_output_length, int pad_rows_zeroed, const float *gscale_dev,
                               void *stream, ScaleTask also_scale = ScaleTask{nullptr, 0});
// pcfgnat_logsoftmax_gather_lse over the [B,T] targets with the eos mask and the force-emit masks; the rows of nodes at
// or beyond a sentence's output length are left unread (zeros in selected and lse)
int lsg_forward_lse_force(const void *logits, int dtype, const int64_t *targets, void *selected, void *lse,
                          const int64_t *output_length, const int64_t *target_length, const unsigned char *matchmask,
                          const unsigned char *keep, int64_t B, int64_t L, int64_t V, int64_t T, void *stream);

// pcfgnat_criterion_loss that also writes the log-likelihoods with the invalid ones zeroed (ll_out [B], may be null)
int criterion_loss_impl(const float *S, const int64_t *target_length, float *out, float *ll_out, int64_t B, int64_t L, int64_t T,
                        int64_t ml, void *stream);

// Settings of pcfgnat_pipeline_config (inside.hip): the most workgroups a pipelined sweep may use (0 = pipelines off) and the
// bound on a block's wait for the one ahead of it, in rounds of polling
int pipeline_max_workgroups();
int pipeline_spin_limit();
// Default bound of a block's wait: 2^15 rounds of a short sleep and one device-scope load, some tens of milliseconds -
// a hundred times the lag of the last block of a sentence behind the first (the blocks of a sentence follow each other
// at about 2 us per block), short enough for a sweep that cannot make progress to fall back without being noticed as a stall.
#define PCFGNAT_DEFAULT_SPIN_LIMIT (1 << 15)
// sentences redone by the one-workgroup Viterbi kernel after their pipelined sweep gave up (viterbi.hip)
int viterbi_redo_count(unsigned long long *count, int reset);

// General max_left (generic_ml.hip)
size_t generic_aux_floats(int64_t B, int64_t L, int64_t T, int64_t ml);
int generic_forward(const float *match_all, const float *links, const int64_t *ol, const int64_t *tl, float *S, float *aux, int64_t B,
                    int64_t L, int64_t T, int64_t ml, void *stream, int skip_ml3_taken = 0);
int generic_backward(const float *go, const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol,
                     const int64_t *tl, float *mg, float *lg, int64_t B, int64_t L, int64_t T, int64_t ml, Seed seed, void *stream, int skip_ml3_taken = 0);
// max_left = 3 with the rules the model can produce (inside_ml3.hip): forward and backward in one launch for the sentences
// that qualify; the others are left to generic_forward / generic_backward with skip_ml3_taken = 1, which skip the rest.
bool inside_ml3_supported(int64_t L, int64_t T);
int inside_ml3_forward_backward(const float *grad_output, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl,
                                float *S, float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, Seed seed,
                                void *stream);
int generic_best_tree(const float *S, float *aux, const float *match_all, const float *links, const int64_t *ol, const int64_t *tl,
                      int64_t *tree, int64_t B, int64_t L, int64_t T, int64_t ml, void *stream);
int generic_viterbi(const float *ob, const float *links, const int64_t *ol, float *S, int64_t *R, int64_t *Lt, int64_t *M, int64_t B,
                    int64_t L, int64_t ml, void *stream, int skip_ml3_taken = 0);
// max_left = 3: whether the tuned kernels are switched on (pcfgnat_max_left3_tuned) and, for the Viterbi tables, whether a
// graph of L nodes fits the one-launch kernel (viterbi.hip); generic_viterbi with skip_ml3_taken = 1 then does the rest.
bool ml3_tuned_on();
bool viterbi_ml3_supported(int64_t L);

// ---- DPP helpers: reductions inside a row of 16 lanes and across a wave64 -------------------------------------
// dpp_ctrl encodings (GFX9): quad_perm = perm bits, row_half_mirror = 0x141, row_mirror = 0x140.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

constexpr int DPP_QUAD_XOR1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// max(v, v of the partner lane) as one DPP instruction.  Written in assembly because fmaxf() on a value that comes out
// of a DPP move (or an LDS load) is compiled to move + canonicalise + max, four instructions in loops that are bound by
// instruction issue; the hardware max already quiets NaNs in the IEEE mode kernels run in.  The leading s_nop covers
// the two wait states a DPP read needs after a VALU write of the same register, which the compiler does not track
// through inline assembly; inputs must not come straight from a transcendental instruction (v_exp/v_log), same reason.
#define PCFGNAT_DPP_MAX(name, ctrl)                                                                          \
    __device__ __forceinline__ float name(float v) {                                                          \
        float r;                                                                                              \
        asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 " ctrl " row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v)); \
        return r;                                                                                             \
    }
PCFGNAT_DPP_MAX(dpp_max_xor1, "quad_perm:[1,0,3,2]")
PCFGNAT_DPP_MAX(dpp_max_xor2, "quad_perm:[2,3,0,1]")
PCFGNAT_DPP_MAX(dpp_max_half_mirror, "row_half_mirror")
PCFGNAT_DPP_MAX(dpp_max_mirror, "row_mirror")
#undef PCFGNAT_DPP_MAX

// All 16 lanes of a DPP row end up with the row's maximum / sum.
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_ROW_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f<DPP_ROW_MIRROR>(v));
    return v;
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f<DPP_QUAD_XOR1>(v);
    v += dpp_f<DPP_QUAD_XOR2>(v);
    v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f<DPP_ROW_MIRROR>(v);
    return v;
}

// Wave64 all-reduce: rows first, then the four row totals through scalar registers.
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (a + b) + (c + d);
}

// Wave64 minimum of an int: DPP inside the rows, the four row results through scalar registers.
__device__ __forceinline__ int wave_min(int v) {
    v = min(v, dpp_i<DPP_QUAD_XOR1>(v));
    v = min(v, dpp_i<DPP_QUAD_XOR2>(v));
    v = min(v, dpp_i<DPP_ROW_HALF_MIRROR>(v));
    v = min(v, dpp_i<DPP_ROW_MIRROR>(v));
    const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return min(min(a, b), min(c, d));
}

__device__ __forceinline__ double wave_max(double v) {
    for (int o = 32; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

constexpr float NEG_INF_F = -__builtin_huge_valf();

// max_left = 3: does this sentence hold a rule through which the loops of pcfg_loss.cu:301-348 could build a composite
// local tree?  Those are links[x, k, c] for the local nodes x = a-3, a-2 in front of every main-chain node a = 5, 9, ...,
// m-1, right children x < c < a, every left option k - twelve per group; the model's link scorer leaves them all -inf
// (a local node has no allowed right child).  Workgroup-uniform result; m must be a valid graph size ((m - 2) % 4 == 0).
template <int NT>
__device__ __forceinline__ bool ml3_composite_rules(const float *__restrict__ links, int L, int m, int tid) {
    const int groups = (m - 2) / 4;
    int found = 0;
    for (int i = tid; i < groups * 12; i += NT) {
        const int gi = i / 12, e = i - gi * 12, a = 4 * gi + 5;
        const int x = e < 8 ? a - 3 : a - 2;
        const int c = e < 8 ? a - 2 + (e >> 2) : a - 1;
        const float v = links[((size_t)x * 4 + (e & 3)) * L + c];
        found |= (v > NEG_INF_F) ? 1 : 0;  // (NaN counts as -inf, as in pcfg_loss.cu:162)
    }
    return __syncthreads_or(found) != 0;
}

// The criterion's reduction (nat_pcfg_loss.py:123-135) by one workgroup of NT threads, in a fixed order:
// out[0] = -(1/B) * sum_b [ll_b finite] ll_b / n_b, out[1] = number of sentences with a non-finite ll_b, where
// ll_b = S[b * stride].  Every thread of the workgroup must call it.
// The criterion's force-emit masking (nat_pcfg_loss.py:116-121) folded into the gather: graph nodes whose input token was
// revealed by glancing (keep[b,p] != 0) may only emit the target position they are aligned to (matchmask[b,s,p] != 0,
// every other position becomes -inf) and pass no gradient to their logits.  keep = null: off.
struct ForceEmit {
    const unsigned char *matchmask;  // [B,T,L]
    const unsigned char *keep;       // [B,L]
};

struct LossTask {
    const float *S;
    const int64_t *tgt_len;
    float *out;  // null: nothing to do
    int B;
    int64_t stride;
    float *ll_out = nullptr;  // [B] or null: the log-likelihoods with the invalid ones (non-finite) zeroed
};

// NT threads form the sum (the order of the additions, and with it the rounding, is a function of NT alone); the
// workgroup may be larger (BLOCK threads), its other threads only keep the barriers company.
template <int NT, int BLOCK = NT>
__device__ __forceinline__ void criterion_loss_block(const LossTask &t) {
    static_assert(BLOCK >= NT, "the workgroup holds at least the threads that sum");
    __shared__ float s_sum[NT];
    __shared__ float s_bad[NT];
    const bool member = BLOCK == NT || (int)threadIdx.x < NT;
    float acc = 0.f, bad = 0.f;
    if (member) {
        for (int b = threadIdx.x; b < t.B; b += NT) {
            const float ll = t.S[(size_t)b * t.stride];
            const bool ok = (ll == ll) && (fabsf(ll) != __builtin_huge_valf());
            if (ok) acc += ll / (float)t.tgt_len[b];
            else bad += 1.f;
            if (t.ll_out != nullptr) t.ll_out[b] = ok ? ll : 0.f;
        }
        s_sum[threadIdx.x] = acc;
        s_bad[threadIdx.x] = bad;
    }
    __syncthreads();
    for (int o = NT / 2; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + o];
            s_bad[threadIdx.x] += s_bad[threadIdx.x + o];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        t.out[0] = -s_sum[0] / (float)t.B;
        t.out[1] = s_bad[0];
    }
}

// Workgroup barrier that orders LDS traffic only: outstanding global stores keep draining in the background instead
// of being waited for (what __syncthreads() does), which matters in sweeps that write a few table cells per step.
// Global data written before it must not be read by other waves after it.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}


// Exchange between the workgroups of one launch (pipelined sweeps): table entries are written once with a device-scope
// store by their owner and polled with device-scope loads by the readers; an all-ones bit pattern, with which the tables
// are filled by an earlier launch, marks an entry that has not arrived.
constexpr unsigned EMPTY32 = 0xFFFFFFFFu;
constexpr unsigned long long EMPTY64 = ~0ull;

__device__ __forceinline__ unsigned long long entry_load(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned entry_load(const unsigned *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void entry_store(unsigned long long *p, double v) {
    __hip_atomic_store(p, (unsigned long long)__double_as_longlong(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void entry_store(unsigned *p, float v) {
    __hip_atomic_store(p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool gave_up(const int *flag) { return __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0; }

}  // namespace pcfgnat
