// Fused log-softmax + target gather over [B*L, V] logits, and its in-place backward.
//
// Replaces logsoftmax_gather_kernel (reference fs_plugins/custom_ops/logsoftmax_gather.cu:238-292), which reads
// every row three times with scalar 2-byte loads, and the two generic torch passes of
// DagLogsoftmaxGatherFunc.backward (fs_plugins/custom_ops/pcfg_loss.py:176-177).
//
// Design (HBM-bound, MI355X): one workgroup per row; the row is fetched once with 16-byte loads and kept in
// registers (chunks beyond the register budget are re-streamed), so HBM sees one read and - when the gradient is
// needed - one write per element.  Row max / sum use DPP wave reductions plus one LDS hop across waves.
//
// Two ways to split the work between forward and backward:
//   * reference split: the forward overwrites the logits with softmax probabilities (read + write), the backward
//     scales them and scatters the target gradients (read + write): four passes over the logits per training step;
//   * log-sum-exp split: the forward only reads (and keeps one log-sum-exp per row), the backward recomputes
//     exp(x - lse) while it writes the gradient (read + write): three passes, and the fp16 gradient is rounded once
//     instead of twice.  The logits must stay untouched between the two calls.
#include "common.hip.h"

namespace pcfgnat {
namespace {

typedef unsigned int vec16 __attribute__((ext_vector_type(4)));  // one 16-byte global access

template <typename T>
struct Elem;
template <>
struct Elem<__half> {
    using compute = float;
    static constexpr int EPV = 8;
    __device__ static __forceinline__ void unpack(const vec16 &v, float *o) {
        const __half2 *h = reinterpret_cast<const __half2 *>(&v);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float2 f = __half22float2(h[i]);
            o[2 * i] = f.x;
            o[2 * i + 1] = f.y;
        }
    }
    __device__ static __forceinline__ vec16 pack(const float *o) {
        vec16 v;
        __half2 *h = reinterpret_cast<__half2 *>(&v);
#pragma unroll
        for (int i = 0; i < 4; i++) h[i] = __floats2half2_rn(o[2 * i], o[2 * i + 1]);
        return v;
    }
    __device__ static __forceinline__ float widen(__half x) { return __half2float(x); }
    __device__ static __forceinline__ __half narrow(float x) { return __float2half_rn(x); }
};
template <>
struct Elem<float> {
    using compute = float;
    static constexpr int EPV = 4;
    __device__ static __forceinline__ void unpack(const vec16 &v, float *o) {
        o[0] = __uint_as_float(v.x);
        o[1] = __uint_as_float(v.y);
        o[2] = __uint_as_float(v.z);
        o[3] = __uint_as_float(v.w);
    }
    __device__ static __forceinline__ vec16 pack(const float *o) {
        vec16 v = {__float_as_uint(o[0]), __float_as_uint(o[1]), __float_as_uint(o[2]), __float_as_uint(o[3])};
        return v;
    }
    __device__ static __forceinline__ float widen(float x) { return x; }
    __device__ static __forceinline__ float narrow(float x) { return x; }
};
template <>
struct Elem<double> {
    using compute = double;
    static constexpr int EPV = 2;
    __device__ static __forceinline__ void unpack(const vec16 &v, double *o) {
        o[0] = __longlong_as_double(((long long)v.y << 32) | v.x);
        o[1] = __longlong_as_double(((long long)v.w << 32) | v.z);
    }
    __device__ static __forceinline__ vec16 pack(const double *o) {
        long long a = __double_as_longlong(o[0]), b = __double_as_longlong(o[1]);
        vec16 v = {(unsigned)a, (unsigned)(a >> 32), (unsigned)b, (unsigned)(b >> 32)};
        return v;
    }
    __device__ static __forceinline__ double widen(double x) { return x; }
    __device__ static __forceinline__ double narrow(double x) { return x; }
};

// Row normalisation: e(v) = exp(v - max) and the row log-sum-exp from sum_v e(v).  In float the subtraction, the change
// of base and the widening of an fp16 input are folded into one fused multiply-add in front of the hardware exp2
// (e(v) = 2^(v*log2e + nb), nb = -max*log2e rounded once; the log-sum-exp undoes exactly that nb, so the rounding of nb
// does not bias the result), which takes the loops below from five VALU instructions per element to two plus the exp2.
template <typename CT>
struct RowNorm;
template <>
struct RowNorm<float> {
    float nb;
    __device__ __forceinline__ explicit RowNorm(float mx) : nb(-mx * 1.4426950408889634f) {}
    __device__ __forceinline__ float e(float v) const { return __builtin_amdgcn_exp2f(__builtin_fmaf(v, 1.4426950408889634f, nb)); }
    __device__ __forceinline__ float lse(float sum) const { return (__builtin_amdgcn_logf(sum) - nb) * 0.6931471805599453f; }
    // v - lse(sum) without the cancellation of two large numbers
    __device__ __forceinline__ float logprob(float v, float sum) const {
        return (__builtin_fmaf(v, 1.4426950408889634f, nb) - __builtin_amdgcn_logf(sum)) * 0.6931471805599453f;
    }
    // exp(v - l) for a given log-sum-exp l
    __device__ static __forceinline__ RowNorm from_lse(float l) { return RowNorm(l); }
};
template <>
struct RowNorm<double> {
    double mx;
    __device__ __forceinline__ explicit RowNorm(double m) : mx(m) {}
    __device__ __forceinline__ double e(double v) const { return exp(v - mx); }
    __device__ __forceinline__ double lse(double sum) const { return mx + log(sum); }
    __device__ __forceinline__ double logprob(double v, double sum) const { return (v - mx) - log(sum); }
    __device__ static __forceinline__ RowNorm from_lse(double l) { return RowNorm(l); }
};

// Running maximum of a row: packed fp16 maxima for half inputs (two elements per instruction, no widening), plain
// compute-type maxima otherwise.
template <typename T>
struct RowMax {
    typename Elem<T>::compute m;
    __device__ __forceinline__ RowMax() : m(-__builtin_huge_val()) {}
    __device__ __forceinline__ void chunk(const vec16 &v) {
        typename Elem<T>::compute o[Elem<T>::EPV];
        Elem<T>::unpack(v, o);
#pragma unroll
        for (int e = 0; e < Elem<T>::EPV; e++) m = (m > o[e] || !(o[e] == o[e])) ? m : o[e];
    }
    __device__ __forceinline__ void scalar(T x) {
        const typename Elem<T>::compute o = Elem<T>::widen(x);
        m = (m > o || !(o == o)) ? m : o;
    }
    __device__ __forceinline__ typename Elem<T>::compute value() const { return m; }
};
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
template <>
struct RowMax<__half> {
    f16x2 m;
    __device__ __forceinline__ RowMax() : m{(_Float16)-__builtin_huge_valf(), (_Float16)-__builtin_huge_valf()} {}
    __device__ __forceinline__ void chunk(const vec16 &v) {
        const f16x2 *h = reinterpret_cast<const f16x2 *>(&v);
#pragma unroll
        for (int i = 0; i < 4; i++) m = __builtin_elementwise_max(m, h[i]);
    }
    __device__ __forceinline__ void scalar(__half x) {
        const _Float16 f = *reinterpret_cast<const _Float16 *>(&x);
        m = __builtin_elementwise_max(m, f16x2{f, f});
    }
    __device__ __forceinline__ float value() const { return fmaxf((float)m.x, (float)m.y); }
};

__device__ __forceinline__ float neg_inf(float) { return -__builtin_huge_valf(); }
__device__ __forceinline__ double neg_inf(double) { return -__builtin_huge_val(); }
__device__ __forceinline__ float vmax(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double vmax(double a, double b) { return fmax(a, b); }

// The logits are streamed: loads and stores are marked non-temporal, with one exception - the forward pass of the
// log-sum-exp split, whose rows the backward pass reads again a few tens of microseconds later.  Ordinary loads leave
// them in the memory-side cache (256 MB on MI355X; non-temporal loads do not allocate there), and the backward, whose
// in-place read+write otherwise runs at the rate of a device copy, finds most of its reads there: measured at 273 MB of
// live rows, forward 51 -> 55 us, backward 101 -> 82 us.
__device__ __forceinline__ vec16 load16(const vec16 *p) { return __builtin_nontemporal_load(p); }
template <bool KEEP>
__device__ __forceinline__ vec16 load16_fwd(const vec16 *p) {
    if (KEEP) return *p;
    return __builtin_nontemporal_load(p);
}
// Makes the compiler forget what it knows about a register-resident chunk, so that each pass re-derives the widened
// values from the packed registers instead of keeping both copies alive (which would halve the occupancy).
__device__ __forceinline__ void opaque(vec16 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void store16(vec16 *p, const vec16 &v) { __builtin_nontemporal_store(v, p); }

// Splits a row that starts at an arbitrary element address into [head scalars][16-byte chunks][tail scalars].
template <typename T>
struct RowSplit {
    int head, nvec, tail;
    __device__ RowSplit(const T *row, int V) {
        constexpr int EPV = Elem<T>::EPV;
        uintptr_t a = reinterpret_cast<uintptr_t>(row);
        int h = (int)(((16 - (a & 15)) & 15) / sizeof(T));
        head = h < V ? h : V;
        nvec = (V - head) / EPV;
        tail = V - head - nvec * EPV;
    }
    // element handled as a scalar by thread `tid` (at most one per thread), or -1
    __device__ int edge_pos(int tid) const {
        if (tid < head) return tid;
        if (tid < head + tail) return head + nvec * Elem<T>::EPV + (tid - head);
        return -1;
    }
};

template <typename CT, int NW>
__device__ __forceinline__ CT block_max(CT v, CT *slots, int wave, int lane) {
    v = wave_max(v);
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    CT r = slots[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r = vmax(r, slots[w]);
    return r;
}
template <typename CT, int NW>
__device__ __forceinline__ CT block_sum(CT v, CT *slots, int wave, int lane) {
    v = wave_sum(v);
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    CT r = slots[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r += slots[w];
    return r;
}

// Launch order of the rows of a [B,L] batch whose sentences use only their first output_length[b] graph nodes: slot k of
// the launch takes the k-th live row (live rows in batch order), the slots behind the last live row take the rows of
// pad nodes, in reverse.  A workgroup of a pad row has next to nothing to do; scattered among the live rows (80 live
// rows, 48 pad rows, 80 live rows, ...) each still holds a workgroup slot for its launch and its first load, which
// at a third of the batch costs the live rows a tenth of the launch; at the end of the grid they run beside the last live
// rows.  Every wave recomputes the map from the lengths: lane i takes sentence i (64 per round), prefix sums inside the
// wave, the sentence found by a ballot.  k is uniform over the wave, so is everything derived from it.
constexpr int COMPACT_MAX_B = 256;
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, true);  // row_shr:1, lanes without a source read 0
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, true);
    const int r0 = __builtin_amdgcn_readlane(v, 15), r1 = __builtin_amdgcn_readlane(v, 31), r2 = __builtin_amdgcn_readlane(v, 47);
    return v + (lane >= 16 ? r0 : 0) + (lane >= 32 ? r1 : 0) + (lane >= 48 ? r2 : 0);
}
struct RowOf {
    int b, p;   // sentence and node
    bool live;  // false: the row of a pad node
};
__device__ __forceinline__ RowOf compact_row(int k, const int64_t *__restrict__ out_len, int B, int L, int lane) {
    RowOf r{0, 0, false};
    // the live rows: sentence by sentence in rounds of 64 (one round for batches of up to 64 sentences)
    int done_live = 0;
    for (int b0 = 0; b0 < B; b0 += 64) {
        int len = 0;
        if (b0 + lane < B) {
            const int64_t v = out_len[b0 + lane];
            len = v < 0 ? 0 : (v > (int64_t)L ? L : (int)v);
        }
        const int live_upto = wave_inclusive_scan(len, lane);
        const int tot_live = __builtin_amdgcn_readlane(live_upto, 63);
        if (k < done_live + tot_live) {  // the first lane whose running count passes k holds the sentence
            const int l = __builtin_ctzll(__ballot(k < done_live + live_upto));
            r.b = b0 + l;
            r.p = k - done_live - __builtin_amdgcn_readlane(live_upto - len, l);
            r.live = true;
            return r;
        }
        done_live += tot_live;
    }
    // behind the live rows: the rows of pad nodes, in reverse (these workgroups have next to nothing to do)
    const int kp = B * L - 1 - k;
    int done_pad = 0;
    for (int b0 = 0; b0 < B; b0 += 64) {
        int len = 0, pad = 0;
        if (b0 + lane < B) {
            const int64_t v = out_len[b0 + lane];
            len = v < 0 ? 0 : (v > (int64_t)L ? L : (int)v);
            pad = L - len;
        }
        const int pad_upto = wave_inclusive_scan(pad, lane);
        const int tot_pad = __builtin_amdgcn_readlane(pad_upto, 63);
        if (kp < done_pad + tot_pad) {
            const int l = __builtin_ctzll(__ballot(kp < done_pad + pad_upto));
            r.b = b0 + l;
            r.p = __builtin_amdgcn_readlane(len, l) + (kp - done_pad - __builtin_amdgcn_readlane(pad_upto - pad, l));
            return r;
        }
        done_pad += tot_pad;
    }
    return r;
}

// The row of a workgroup.  The launch is a grid of (L, min(B, 65535), ceil(B / 65535)) workgroups, so sentence and node
// come out of the workgroup index without a division (a 64-bit division by a run-time L is some hundred scalar
// instructions in front of the row's first load).  mode 2: the workgroup's running number selects the k-th live row.
__device__ __forceinline__ bool row_of_workgroup(int mode, const int64_t *__restrict__ out_len, int B, int L, int lane, RowOf &r) {
    const int b = (int)blockIdx.z * 65535 + (int)blockIdx.y;
    if (b >= B) return false;
    if (mode == 2) {
        r = compact_row(b * L + (int)blockIdx.x, out_len, B, L, lane);
    } else {
        r.b = b;
        r.p = (int)blockIdx.x;
        r.live = mode == 0 || (int64_t)r.p < out_len[b];
    }
    return true;
}

// First position, among the elements this thread holds, whose value equals the row maximum (0x7fffffff if none).
template <typename T, int NT, int MAXC>
__device__ __forceinline__ int first_pos_of_max(const vec16 (&buf)[MAXC], const RowSplit<T> &sp, const vec16 *xv, int tid, int ep,
                                                typename Elem<T>::compute edge, typename Elem<T>::compute mx) {
    using CT = typename Elem<T>::compute;
    constexpr int EPV = Elem<T>::EPV;
    int first = 0x7fffffff;
    if (ep >= 0 && edge == mx) first = ep;
#pragma unroll
    for (int i = 0; i < MAXC; i++) {
        const int c = tid + i * NT;
        if (c < sp.nvec) {
            CT v[EPV];
            Elem<T>::unpack(buf[i], v);
#pragma unroll
            for (int e = EPV - 1; e >= 0; e--)
                if (v[e] == mx) first = min(first, sp.head + c * EPV + e);
        }
    }
    for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) {
        CT v[EPV];
        Elem<T>::unpack(load16(xv + c), v);
#pragma unroll
        for (int e = EPV - 1; e >= 0; e--)
            if (v[e] == mx) first = min(first, sp.head + c * EPV + e);
    }
    return first;
}

// NT threads; up to MAXC 16-byte chunks per thread stay in registers, GMAX gathered targets per thread.  KEEP: the rows
// are read again soon (see load16_fwd).
template <typename T, int NT, int MAXC, int GMAX, bool GRAD, bool KEEP>
__global__ __launch_bounds__(NT) void lsg_fwd_kernel(T *__restrict__ x, const int64_t *__restrict__ idx, int64_t sb,
                                                     int64_t sl, int64_t st,
                                                     typename Elem<T>::compute *__restrict__ sel, int B, int L,
                                                     int V, int Tn, const int64_t *__restrict__ eos_out_len,
                                                     const int64_t *__restrict__ eos_tgt_len,
                                                     typename Elem<T>::compute *__restrict__ lse_out,
                                                     int64_t *__restrict__ argmax_out, ForceEmit fe, int skip_pad_rows) {
    using CT = typename Elem<T>::compute;
    constexpr int EPV = Elem<T>::EPV;
    constexpr int NW = NT / 64;
    __shared__ CT s_max[NW];
    __shared__ CT s_sum[NW];
    __shared__ int s_arg;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    {
        // One row per workgroup.  Rows of nodes beyond the sentence's graph (pads) feed nothing downstream of the
        // criterion: neither sweep reads them and their gradient is zero.  When asked to, leave them unread and define
        // their outputs as zeros (skip_pad_rows = 1: rows in batch order; 2: live rows first, see compact_row).
        RowOf at;
        if (!row_of_workgroup(skip_pad_rows, eos_out_len, B, L, lane, at)) return;
        const int64_t row = (int64_t)at.b * L + at.p;
        const bool pad_row = !at.live;  // workgroup-uniform
        T *xr = x + row * (int64_t)V;
        if (pad_row) {
            for (int s2 = tid; s2 < Tn; s2 += NT) sel[row * (int64_t)Tn + s2] = (CT)0;
            if (tid == 0) {
                if (lse_out != nullptr) lse_out[row] = (CT)0;
                if (argmax_out != nullptr) argmax_out[row] = 0;
            }
            return;
        }
        const RowSplit<T> sp(xr, V);
        const vec16 *xv = reinterpret_cast<const vec16 *>(xr + sp.head);

        // Load order: target indices, then the whole row, then the gathered logits.  The gathers depend on the indices;
        // issued before the row they would hold its loads back by one memory round trip per row.  They still complete
        // before anything is stored to the row (the stores come after two workgroup reductions over the loaded data).
        int64_t tg[GMAX];
        {
            const int64_t *ir = idx + at.b * sb + at.p * sl;
#pragma unroll
            for (int g = 0; g < GMAX; g++) {
                const int s = tid + g * NT;
                tg[g] = (s < Tn) ? ir[(int64_t)s * st] : 0;
            }
        }
        vec16 buf[MAXC];
#pragma unroll
        for (int i = 0; i < MAXC; i++) {
            int c = tid + i * NT;
            if (c < sp.nvec) buf[i] = load16_fwd<KEEP>(xv + c);
        }
        const int ep = sp.edge_pos(tid);
        CT edge = neg_inf(CT());
        if (ep >= 0) edge = Elem<T>::widen(xr[ep]);
        CT gv[GMAX];
#pragma unroll
        for (int g = 0; g < GMAX; g++) {
            const int s = tid + g * NT;
            gv[g] = 0;
            if (s < Tn) gv[g] = ((uint64_t)tg[g] < (uint64_t)V) ? Elem<T>::widen(xr[tg[g]]) : (CT)NAN;
        }

        // ---- max
        RowMax<T> rmax;
        if (ep >= 0) rmax.scalar(xr[ep]);
#pragma unroll
        for (int i = 0; i < MAXC; i++)
            if (tid + i * NT < sp.nvec) rmax.chunk(buf[i]);
        for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) rmax.chunk(load16_fwd<KEEP>(xv + c));
        if (argmax_out != nullptr && tid == 0) s_arg = 0x7fffffff;
        const CT mine = rmax.value();
        const CT mx = block_max<CT, NW>(mine, s_max, wave, lane);  // barrier inside
        const RowNorm<CT> rn(mx);
#pragma unroll
        for (int i = 0; i < MAXC; i++) opaque(buf[i]);
        // optional arg max of the row (first maximum): found by the threads whose own maximum is the row's
        if (argmax_out != nullptr && mine == mx) atomicMin(&s_arg, first_pos_of_max<T, NT, MAXC>(buf, sp, xv, tid, ep, edge, mx));

        // ---- sum of exp
        CT sum = (ep >= 0) ? rn.e(edge) : (CT)0;
#pragma unroll
        for (int i = 0; i < MAXC; i++) {
            if (tid + i * NT < sp.nvec) {
                CT v[EPV];
                Elem<T>::unpack(buf[i], v);
#pragma unroll
                for (int e = 0; e < EPV; e++) sum += rn.e(v[e]);
            }
        }
        for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) {
            CT v[EPV];
            Elem<T>::unpack(load16_fwd<KEEP>(xv + c), v);
#pragma unroll
            for (int e = 0; e < EPV; e++) sum += rn.e(v[e]);
        }
        sum = block_sum<CT, NW>(sum, s_sum, wave, lane);
        const CT row_lse = rn.lse(sum);  // (the reduction's barrier also completes s_arg)
        if (lse_out != nullptr && tid == 0) lse_out[row] = row_lse;
        if (argmax_out != nullptr && tid == 0) argmax_out[row] = (s_arg == 0x7fffffff) ? 0 : s_arg;
#pragma unroll
        for (int i = 0; i < MAXC; i++) opaque(buf[i]);

        // optional fused eos mask (nat_pcfg_loss.py:111-115): only the last graph node may emit the last target token
        int eos_col = -1;
        if (eos_out_len != nullptr) {
            if (at.p != eos_out_len[at.b] - 1) eos_col = (int)(eos_tgt_len[at.b] - 1);
        }
        const bool forced = fe.keep != nullptr && fe.keep[row] != 0;  // (nat_pcfg_loss.py:116-121)
#pragma unroll
        for (int g = 0; g < GMAX; g++) {
            int s = tid + g * NT;
            if (s < Tn) {
                CT val = (s == eos_col) ? neg_inf(CT()) : rn.logprob(gv[g], sum);
                if (forced && fe.matchmask[((int64_t)at.b * Tn + s) * L + at.p] == 0) val = neg_inf(CT());
                sel[row * (int64_t)Tn + s] = val;
            }
        }

        if (GRAD) {
            const CT inv = (CT)1 / sum;
            vec16 *xw = reinterpret_cast<vec16 *>(xr + sp.head);
#pragma unroll
            for (int i = 0; i < MAXC; i++) {
                int c = tid + i * NT;
                if (c < sp.nvec) {
                    CT v[EPV];
                    Elem<T>::unpack(buf[i], v);
#pragma unroll
                    for (int e = 0; e < EPV; e++) v[e] = rn.e(v[e]) * inv;
                    store16(xw + c, Elem<T>::pack(v));
                }
            }
            for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) {
                CT v[EPV];
                Elem<T>::unpack(load16_fwd<KEEP>(xv + c), v);
#pragma unroll
                for (int e = 0; e < EPV; e++) v[e] = rn.e(v[e]) * inv;
                store16(xw + c, Elem<T>::pack(v));
            }
            if (ep >= 0) xr[ep] = Elem<T>::narrow(rn.e(edge) * inv);
        }
    }
}

// Decode front-end: best token of every row and its log-probability, max_v log_softmax(x)[v] and the first arg max
// (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-415), in one read of the logits instead of materialising the
// log-softmax.  Same row-in-registers structure as the gather forward; the position of the maximum is recovered by
// the (usually single) thread whose own maximum equals the row's.
template <typename T, int NT, int MAXC>
__global__ __launch_bounds__(NT) void ls_max_kernel(const T *__restrict__ x, typename Elem<T>::compute *__restrict__ best_lprob,
                                                    int64_t *__restrict__ best_idx, int64_t rows, int V) {
    using CT = typename Elem<T>::compute;
    constexpr int EPV = Elem<T>::EPV;
    constexpr int NW = NT / 64;
    __shared__ CT s_max[NW];
    __shared__ CT s_sum[NW];
    __shared__ int s_arg;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    {
        const int64_t row = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;  // one row per workgroup
        if (row >= rows) return;
        const T *xr = x + row * (int64_t)V;
        const RowSplit<T> sp(xr, V);
        const vec16 *xv = reinterpret_cast<const vec16 *>(xr + sp.head);
        vec16 buf[MAXC];
#pragma unroll
        for (int i = 0; i < MAXC; i++) {
            int c = tid + i * NT;
            if (c < sp.nvec) buf[i] = load16(xv + c);
        }
        const int ep = sp.edge_pos(tid);
        CT edge = neg_inf(CT());
        if (ep >= 0) edge = Elem<T>::widen(xr[ep]);
        if (tid == 0) s_arg = 0x7fffffff;

        RowMax<T> rmax;
        if (ep >= 0) rmax.scalar(xr[ep]);
#pragma unroll
        for (int i = 0; i < MAXC; i++)
            if (tid + i * NT < sp.nvec) rmax.chunk(buf[i]);
        for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) rmax.chunk(load16(xv + c));
        const CT mine = rmax.value();
        const CT mx = block_max<CT, NW>(mine, s_max, wave, lane);  // barrier inside: s_arg is initialised
        const RowNorm<CT> rn(mx);
#pragma unroll
        for (int i = 0; i < MAXC; i++) opaque(buf[i]);

        if (mine == mx) atomicMin(&s_arg, first_pos_of_max<T, NT, MAXC>(buf, sp, xv, tid, ep, edge, mx));

        CT sum = (ep >= 0) ? rn.e(edge) : (CT)0;
#pragma unroll
        for (int i = 0; i < MAXC; i++) {
            if (tid + i * NT < sp.nvec) {
                CT v[EPV];
                Elem<T>::unpack(buf[i], v);
#pragma unroll
                for (int e = 0; e < EPV; e++) sum += rn.e(v[e]);
            }
        }
        for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) {
            CT v[EPV];
            Elem<T>::unpack(load16(xv + c), v);
#pragma unroll
            for (int e = 0; e < EPV; e++) sum += rn.e(v[e]);
        }
        sum = block_sum<CT, NW>(sum, s_sum, wave, lane);  // barrier inside: s_arg is final
        if (tid == 0) {
            best_lprob[row] = rn.logprob(mx, sum);
            // a row whose maximum is NaN-free but never found (all NaN) keeps index 0, like an all-equal row
            best_idx[row] = (s_arg == 0x7fffffff) ? 0 : s_arg;
        }
    }
}

// In-place backward.  TCAP = most targets per row handled through LDS; up to MAXC chunks per thread are in flight.
// FROM_LOGITS = false: the buffer holds the probabilities the forward left (reference split, with the reference's
// roundings to the buffer dtype); true: it holds the untouched logits and `lse` the row log-sum-exps.
//
// Every element of the row becomes p * (-sum_s g[s]); the (at most T) target columns also receive their g[s]
// (scatter_add_, pcfg_loss.py:177: duplicates of a column accumulate in order).  Every 16-byte chunk is loaded once and
// stored once, by the thread that streams it: the thread of a target posts (target, chunk slot, element) into the
// streaming thread's mailbox in LDS (BOX entries per thread, taken in the order of arrival and sorted by target before
// use, so that duplicates of a column are added in the order of the targets whatever the arrival order was); a thread
// whose mailbox overflowed goes through all targets for each of its chunks instead.  No second load, no store beside
// the row's own stream: as a take-over of such chunks by the targets' threads (a second, dependent load per target,
// a 16-byte store of its own and a hole in the stream's stores) the same work took 123 instead of 95-100 us at 140
// targets per row, of which the scattered stores were 8 us, the holes 7 us and the second loads 5 us (each switched
// off in turn).
template <typename T, int NT, int MAXC, int TCAP, bool FROM_LOGITS>
__global__ __launch_bounds__(NT, FROM_LOGITS ? 1 : 6) void lsg_bwd_kernel(T *__restrict__ p, const int64_t *__restrict__ idx, int64_t sb,
                                                     int64_t sl, int64_t st,
                                                     const typename Elem<T>::compute *__restrict__ gsel, int B,
                                                     int L, int V, int Tn,
                                                     const typename Elem<T>::compute *__restrict__ lse, LossTask loss,
                                                     const unsigned char *__restrict__ detach_rows,
                                                     const int64_t *__restrict__ pad_out_len, int pad_mode,
                                                     int pad_rows_zeroed, const float *__restrict__ gscale_dev, ScaleTask also_scale) {
    using CT = typename Elem<T>::compute;
    constexpr int EPV = Elem<T>::EPV;
    constexpr int FIX = (TCAP + NT - 1) / NT;
    constexpr int BOX = 4;                      // mailbox entries per streaming thread
    constexpr unsigned EDGE_BIT = 1u << 30;     // in the mailbox count: a target points at this thread's element outside the chunks
    constexpr unsigned COUNT_MASK = 0xFFFFu;
    constexpr int SLOT_SHIFT = 16;              // above the count: one bit per chunk slot (bit MAXC: any chunk beyond them) that holds
                                                // a target which found the mailbox full
    static_assert(SLOT_SHIFT + MAXC < 30, "the slot bits end below EDGE_BIT");
    constexpr unsigned NO_ENTRY = 0xFFFFFFFFu;  // sorts behind every entry; its slot field matches no slot
    static_assert(MAXC <= 30, "one bit per register-resident chunk");
    static_assert(TCAP <= 1024, "a target index takes ten bits of a mailbox entry");
    // an upstream factor of the whole gradient that only the device knows (the loss's own upstream gradient under fp16 loss
    // scaling): folded into g in the compute type, ahead of the single rounding to the buffer's dtype (pcfg_loss.py:77-83,
    // 176-177 scale g before the cast as well)
    const CT gs = (FROM_LOGITS && gscale_dev != nullptr) ? (CT)*gscale_dev : (CT)1;
    if (loss.out != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) criterion_loss_block<NT>(loss);  // workgroup-uniform
    __shared__ __attribute__((aligned(16))) int s_idx[TCAP + 4];  // target column of position s, -1 if out of range; padded
                                                                  // to a multiple of four with -2 (matches nothing)
    __shared__ CT s_g[TCAP];         // g[s], zero for a detached row
    __shared__ unsigned s_cnt[NT];   // per thread: how many targets point into its chunks (and EDGE_BIT)
    __shared__ __attribute__((aligned(16))) unsigned s_box[NT * BOX];  // (target << 16) | (chunk slot << 4) | element
    const int tid = threadIdx.x, lane = tid & 63;

    if (also_scale.p != nullptr && gscale_dev != nullptr) {  // a side task spread over every thread of the launch
        const size_t slot = ((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        const size_t total = (size_t)gridDim.x * gridDim.y * gridDim.z * NT;
        const float sc = *gscale_dev;
        for (size_t i = slot * NT + tid; i < also_scale.n; i += total) also_scale.p[i] *= sc;
    }
    // One row per workgroup.  Rows of nodes beyond the sentence's graph (pads) get no gradient from the criterion, whose
    // backward sweep leaves their upstream gradient all zero: p * 0 plus zeros is zero whatever the row holds, so such a
    // row is written without being read (pad_mode = 1: rows in batch order, the lengths come through the scalar cache; 2:
    // live rows first, see compact_row).
    RowOf at;
    if (!row_of_workgroup(pad_mode, pad_out_len, B, L, lane, at)) return;
    const int64_t row = (int64_t)at.b * L + at.p;
    const bool pad_row = !at.live;  // workgroup-uniform
    T *pr = p + row * (int64_t)V;
    const RowSplit<T> sp(pr, V);
    vec16 *pv = reinterpret_cast<vec16 *>(pr + sp.head);
    const int ep = sp.edge_pos(tid);
    if (pad_row) {
        if (pad_rows_zeroed) return;  // an earlier launch of the caller has written the zeros
        vec16 z;
        z.x = z.y = z.z = z.w = 0;
        for (int c = tid; c < sp.nvec; c += NT) store16(pv + c, z);
        if (ep >= 0) pr[ep] = Elem<T>::narrow((CT)0);
        return;
    }

    // The small per-row inputs are requested first (independent loads, no chain), the row's chunks right behind them.
    const CT *gr = gsel + row * (int64_t)Tn;
    const int64_t *ir = idx + at.b * sb + at.p * sl;
    // a row whose gathered values were detached (force-emit, nat_pcfg_loss.py:121) gets no gradient at all
    unsigned char detached = 0;
    if (detach_rows != nullptr) detached = detach_rows[row];
    int64_t tcol[FIX];
    CT tg[FIX];
#pragma unroll
    for (int r = 0; r < FIX; r++) {
        const int s = tid + r * NT;
        tcol[r] = -1;
        tg[r] = 0;
        if (s < Tn) {
            tcol[r] = ir[(int64_t)s * st];
            tg[r] = gr[s];
        }
    }
    CT row_lse = 0;
    if (FROM_LOGITS) row_lse = lse[row];

    vec16 buf[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; i++) {
        int c = tid + i * NT;
        if (c < sp.nvec) buf[i] = load16(pv + c);
    }
    T edge_raw = Elem<T>::narrow((CT)0);
    if (ep >= 0) edge_raw = pr[ep];

    s_cnt[tid] = 0;
#pragma unroll
    for (int r = 0; r < FIX; r++) {
        const int s = tid + r * NT;
        if (s < ((Tn + 3) & ~3)) {
            s_idx[s] = s >= Tn ? -2 : ((uint64_t)tcol[r] < (uint64_t)V) ? (int)tcol[r] : -1;
            if (s < Tn) s_g[s] = detached ? (CT)0 : tg[r];
        }
    }
    lds_barrier();

    // The threads of the targets post them to the threads that stream their chunks.
    const int body_end = sp.head + sp.nvec * EPV;  // columns [head, body_end) travel as 16-byte chunks
#pragma unroll
    for (int r = 0; r < FIX; r++) {
        const int s = tid + r * NT;
        if (s < Tn && (uint64_t)tcol[r] < (uint64_t)V) {
            const int col = (int)tcol[r];
            if (col < sp.head) {
                atomicOr(&s_cnt[col], EDGE_BIT);
            } else if (col >= body_end) {
                atomicOr(&s_cnt[sp.head + (col - body_end)], EDGE_BIT);
            } else {
                const int cc = (col - sp.head) / EPV, e = (col - sp.head) - cc * EPV, owner = cc % NT;
                const unsigned at = atomicAdd(&s_cnt[owner], 1u) & COUNT_MASK;
                if (at < (unsigned)BOX) s_box[owner * BOX + at] = ((unsigned)s << 16) | ((unsigned)(cc / NT) << 4) | (unsigned)e;
                else atomicOr(&s_cnt[owner], 1u << (SLOT_SHIFT + min(cc / NT, MAXC)));  // no room: at least which chunk it is
            }
        }
    }
    lds_barrier();
    const unsigned posted = s_cnt[tid];
    const int count = (int)(posted & COUNT_MASK);
    const bool overflow = count > BOX;  // (then every target is looked at for every chunk that holds one)
    // bit i: an entry for the chunk of slot i; bit 31: one for a chunk beyond the register-resident ones.  The entries
    // themselves stay in LDS (sorted by target, the high bits, where there are several) and are read again by the few
    // threads that have any, chunk by chunk: held in registers they cost the kernel its third workgroup per compute unit.
    unsigned mine = 0;
    uint4 *my_box = reinterpret_cast<uint4 *>(s_box) + tid;
    if (count > 0) {
        uint4 q = *my_box;
        q.y = count > 1 ? q.y : NO_ENTRY;
        q.z = count > 2 ? q.z : NO_ENTRY;
        q.w = count > 3 ? q.w : NO_ENTRY;
        auto order = [](unsigned &x, unsigned &y) {
            const unsigned lo = min(x, y), hi = max(x, y);
            x = lo;
            y = hi;
        };
        if (count > 1) {  // a sorting network of five exchanges
            order(q.x, q.y);
            order(q.z, q.w);
            order(q.x, q.z);
            order(q.y, q.w);
            order(q.y, q.z);
        }
        *my_box = q;  // (sorted, the unused entries marked)
        const unsigned e[BOX] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int k = 0; k < BOX; k++)
            if (e[k] != NO_ENTRY) mine |= ((e[k] >> 4) & 0xFFFu) < (unsigned)MAXC ? 1u << ((e[k] >> 4) & 0xFFFu) : 1u << 31;
        const unsigned late = (posted >> SLOT_SHIFT) & ((2u << MAXC) - 1u);
        mine |= (late & ((1u << MAXC) - 1u)) | ((late >> MAXC) << 31);
    }
    // -(sum_s g), computed redundantly by every wave; rounded to the buffer dtype in the reference split (pcfg_loss.py:176)
    CT part = 0;
    for (int s = lane; s < Tn; s += 64) part += s_g[s];
    const CT ns = FROM_LOGITS ? -wave_sum(part) * gs : Elem<T>::widen(Elem<T>::narrow(-wave_sum(part)));
    const RowNorm<CT> rn = RowNorm<CT>::from_lse(row_lse);
    // the gradient of position u as it is added to its column
    auto g_at = [&](int u) -> CT { return FROM_LOGITS ? s_g[u] * gs : Elem<T>::widen(Elem<T>::narrow(s_g[u])); };
    // v[0..n) hold p * ns for columns col0 .. col0+n-1: add the gradients of targets u0, u0+1, ... < u1 that point there
    auto add_targets = [&](CT *v, int n, int col0, int u0, int u1) {
        for (int u = u0; u < u1; u++) {
            const int e = s_idx[u] - col0;
            if ((unsigned)e >= (unsigned)n) continue;
            const CT g = g_at(u);
#pragma unroll
            for (int k = 0; k < EPV; k++)
                if (k < n && k == e) v[k] = FROM_LOGITS ? v[k] + g : Elem<T>::widen(Elem<T>::narrow(v[k] + g));
        }
    };
    // v[] holds p * ns of the chunk in slot `slot`: the posted targets of that chunk, in their order
    auto add_posted = [&](CT *v, int slot) {
        const uint4 q = *my_box;
        const unsigned box[BOX] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int k = 0; k < BOX; k++) {
            if (((box[k] >> 4) & 0xFFFu) == (unsigned)slot) {
                const int e = (int)(box[k] & 15u);
                const CT g = g_at((int)(box[k] >> 16));
#pragma unroll
                for (int j = 0; j < EPV; j++)
                    if (j == e) v[j] = FROM_LOGITS ? v[j] + g : Elem<T>::widen(Elem<T>::narrow(v[j] + g));
            }
        }
    };

#pragma unroll
    for (int i = 0; i < MAXC; i++) {
        int c = tid + i * NT;
        if (c < sp.nvec) {
            CT v[EPV];
            Elem<T>::unpack(buf[i], v);
#pragma unroll
            for (int e = 0; e < EPV; e++) v[e] = (FROM_LOGITS ? rn.e(v[e]) : v[e]) * ns;
            if (mine & (1u << i)) {
                if (!FROM_LOGITS) {  // p * ns is rounded before the adds
#pragma unroll
                    for (int e = 0; e < EPV; e++) v[e] = Elem<T>::widen(Elem<T>::narrow(v[e]));
                }
                if (overflow) add_targets(v, EPV, sp.head + c * EPV, 0, Tn);
                else add_posted(v, i);
            }
            store16(pv + c, Elem<T>::pack(v));
        }
    }
    for (int c = tid + MAXC * NT; c < sp.nvec; c += NT) {
        CT v[EPV];
        Elem<T>::unpack(load16(pv + c), v);
#pragma unroll
        for (int e = 0; e < EPV; e++) v[e] = (FROM_LOGITS ? rn.e(v[e]) : v[e]) * ns;
        if (mine & (1u << 31)) {
            if (!FROM_LOGITS) {
#pragma unroll
                for (int e = 0; e < EPV; e++) v[e] = Elem<T>::widen(Elem<T>::narrow(v[e]));
            }
            if (overflow) add_targets(v, EPV, sp.head + c * EPV, 0, Tn);
            else add_posted(v, c / NT);
        }
        store16(pv + c, Elem<T>::pack(v));
    }
    if (ep >= 0) {  // unaligned rows: the elements in front of and behind the 16-byte chunks, one per thread
        CT v = (FROM_LOGITS ? rn.e(Elem<T>::widen(edge_raw)) : Elem<T>::widen(edge_raw)) * ns;
        if (posted & EDGE_BIT) {
            if (!FROM_LOGITS) v = Elem<T>::widen(Elem<T>::narrow(v));
            add_targets(&v, 1, ep, 0, Tn);
        }
        pr[ep] = Elem<T>::narrow(v);
    }
}

// One workgroup per row: the rows along x, folded over y beyond 2^30 of them.
inline dim3 row_grid(int64_t rows) {
    const int64_t gx = rows < (1LL << 30) ? rows : (1LL << 30);
    return dim3((unsigned)gx, (unsigned)((rows + gx - 1) / gx));
}
// One workgroup per (node, sentence): see row_of_workgroup.
inline dim3 node_sentence_grid(int64_t B, int L) {
    const int64_t gy = B < 65535 ? B : 65535;
    return dim3((unsigned)L, (unsigned)gy, (unsigned)((B + gy - 1) / gy));
}

// How a launch that leaves out the rows of pad nodes orders its rows: 2 = live rows first (batches of up to COMPACT_MAX_B
// sentences whose row count fits an int), 1 = batch order.
inline int pad_row_mode(int64_t rows, int L) { return (rows / L <= COMPACT_MAX_B && rows < (1LL << 30)) ? 2 : 1; }

template <typename T>
int launch_fwd(void *x, const int64_t *idx, int64_t sb, int64_t sl, int64_t st, void *sel, int grad, int64_t B,
               int L, int V, int Tn, const int64_t *eos_ol, const int64_t *eos_tl, void *lse, int64_t *argmax, hipStream_t stream,
               ForceEmit fe = ForceEmit{nullptr, nullptr}, int skip_pad_rows = 0) {
    using CT = typename Elem<T>::compute;
    constexpr int NT = 512;
    // 10 chunks x 512 threads x 16 B = 80 KB of a row in registers: a 40k-entry fp16 row exactly, half of an fp32 one.
    constexpr int MAXC = 5120 / NT;
    constexpr int GMAX = 1024 / NT;
    if (Tn > NT * GMAX) return fail(PCFGNAT_EUNSUPPORTED, "logsoftmax_gather: T=%d exceeds %d targets per row", Tn, NT * GMAX);
    PCFGNAT_REQUIRE(B * L < (1LL << 31) && B < 65535LL * 65535LL, "logsoftmax_gather: %lld rows exceed what one launch indexes",
                    (long long)(B * L));
    const dim3 grid = node_sentence_grid(B, L);
    if (skip_pad_rows) skip_pad_rows = pad_row_mode(B * L, L);
    if (grad)
        hipLaunchKernelGGL((lsg_fwd_kernel<T, NT, MAXC, GMAX, true, false>), grid, dim3(NT), 0, stream, (T *)x, idx, sb,
                           sl, st, (CT *)sel, (int)B, L, V, Tn, eos_ol, eos_tl, (CT *)lse, argmax, fe, skip_pad_rows);
    else if (lse != nullptr)  // log-sum-exp split: the backward pass over the same rows follows
        hipLaunchKernelGGL((lsg_fwd_kernel<T, NT, MAXC, GMAX, false, true>), grid, dim3(NT), 0, stream, (T *)x, idx,
                           sb, sl, st, (CT *)sel, (int)B, L, V, Tn, eos_ol, eos_tl, (CT *)lse, argmax, fe, skip_pad_rows);
    else
        hipLaunchKernelGGL((lsg_fwd_kernel<T, NT, MAXC, GMAX, false, false>), grid, dim3(NT), 0, stream, (T *)x, idx,
                           sb, sl, st, (CT *)sel, (int)B, L, V, Tn, eos_ol, eos_tl, (CT *)lse, argmax, fe, skip_pad_rows);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

template <typename T>
int launch_bwd(void *p, const int64_t *idx, int64_t sb, int64_t sl, int64_t st, const void *g, int64_t B, int L, int V,
               int Tn, const void *lse, const LossTask &loss, hipStream_t stream, const unsigned char *detach_rows = nullptr,
               const int64_t *pad_out_len = nullptr, int pad_rows_zeroed = 0, const float *gscale_dev = nullptr,
               ScaleTask also_scale = ScaleTask{nullptr, 0}) {
    using CT = typename Elem<T>::compute;
    constexpr int NT = 512;
    constexpr int MAXC = 10;
    constexpr int TCAP = 1024;  // most targets per row; up to NT of them the kernel with one target per thread (fewer registers)
    if (Tn > TCAP) return fail(PCFGNAT_EUNSUPPORTED, "logsoftmax_gather_backward: T=%d exceeds %d targets per row", Tn, TCAP);
    PCFGNAT_REQUIRE(B * L < (1LL << 31) && B < 65535LL * 65535LL, "logsoftmax_gather_backward: %lld rows exceed what one launch indexes",
                    (long long)(B * L));
    const dim3 grid = node_sentence_grid(B, L);
    const int pad_mode = pad_out_len == nullptr ? 0 : pad_row_mode(B * L, L);
#define PCFGNAT_LSG_BWD(tcap)                                                                                                              \
    do {                                                                                                                                   \
        if (lse != nullptr)                                                                                                                \
            hipLaunchKernelGGL((lsg_bwd_kernel<T, NT, MAXC, tcap, true>), grid, dim3(NT), 0, stream, (T *)p, idx, sb, sl, st,              \
                               (const CT *)g, (int)B, L, V, Tn, (const CT *)lse, loss, detach_rows, pad_out_len, pad_mode, pad_rows_zeroed, \
                               gscale_dev, also_scale);                                                                                    \
        else                                                                                                                               \
            hipLaunchKernelGGL((lsg_bwd_kernel<T, NT, MAXC, tcap, false>), grid, dim3(NT), 0, stream, (T *)p, idx, sb, sl, st,             \
                               (const CT *)g, (int)B, L, V, Tn, (const CT *)nullptr, loss, detach_rows, pad_out_len, pad_mode,             \
                               pad_rows_zeroed, nullptr, ScaleTask{nullptr, 0});                                                           \
    } while (0)
    if (Tn <= NT) PCFGNAT_LSG_BWD(NT);
    else PCFGNAT_LSG_BWD(TCAP);
#undef PCFGNAT_LSG_BWD
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

template <typename T>
int launch_ls_max(const void *x, void *best_lprob, int64_t *best_idx, int64_t rows, int V, hipStream_t stream) {
    using CT = typename Elem<T>::compute;
    constexpr int NT = 512;
    constexpr int MAXC = 10;
    const dim3 grid = row_grid(rows);
    hipLaunchKernelGGL((ls_max_kernel<T, NT, MAXC>), grid, dim3(NT), 0, stream, (const T *)x, (CT *)best_lprob, best_idx,
                       rows, V);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

int check_common(const void *x, const int64_t *idx, const void *o, int64_t B, int64_t L, int64_t V, int64_t T) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 0 && V >= 1 && T >= 0, "logsoftmax_gather: negative or empty dimension (B=%lld L=%lld V=%lld T=%lld)",
                    (long long)B, (long long)L, (long long)V, (long long)T);
    PCFGNAT_REQUIRE(V < (1LL << 31) && T < (1LL << 31) && L < (1LL << 31), "logsoftmax_gather: V, T, L must fit in int32");
    if (B * L == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(x != nullptr && o != nullptr && (idx != nullptr || T == 0), "logsoftmax_gather: null pointer");
    return PCFGNAT_OK;
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

static int lsg_forward_dispatch(void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl, int64_t st,
                                void *selected, int require_grad, int64_t B, int64_t L, int64_t V, int64_t T,
                                const int64_t *eos_ol, const int64_t *eos_tl, void *lse, void *stream, int64_t *argmax = nullptr,
                                ForceEmit fe = ForceEmit{nullptr, nullptr}, int skip_pad_rows = 0) {
    int rc = check_common(word_ins_out, select_idx, selected, B, L, V, T);
    if (rc != PCFGNAT_OK) return rc;
    if (B * L == 0) return PCFGNAT_OK;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case PCFGNAT_F16:
            return launch_fwd<__half>(word_ins_out, select_idx, sb, sl, st, selected, require_grad, B, (int)L, (int)V, (int)T, eos_ol, eos_tl, lse, argmax, s, fe, skip_pad_rows);
        case PCFGNAT_F32:
            return launch_fwd<float>(word_ins_out, select_idx, sb, sl, st, selected, require_grad, B, (int)L, (int)V, (int)T, eos_ol, eos_tl, lse, argmax, s, fe, skip_pad_rows);
        case PCFGNAT_F64:
            return launch_fwd<double>(word_ins_out, select_idx, sb, sl, st, selected, require_grad, B, (int)L, (int)V, (int)T, eos_ol, eos_tl, lse, argmax, s, fe, skip_pad_rows);
        default:
            return fail(PCFGNAT_EINVAL, "logsoftmax_gather: unknown dtype code %d (float16, float32, float64 are dispatched)", dtype);
    }
}

extern "C" int pcfgnat_logsoftmax_gather(void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl,
                                         int64_t st, void *selected, int require_grad, int64_t B, int64_t L, int64_t V,
                                         int64_t T, void *stream) {
    return lsg_forward_dispatch(word_ins_out, dtype, select_idx, sb, sl, st, selected, require_grad, B, L, V, T, nullptr, nullptr,
                                nullptr, stream);
}

extern "C" int pcfgnat_logsoftmax_gather_eos(void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl,
                                             int64_t st, void *selected, int require_grad, const int64_t *output_length,
                                             const int64_t *target_length, int64_t B, int64_t L, int64_t V, int64_t T,
                                             void *stream) {
    PCFGNAT_REQUIRE(B == 0 || (output_length && target_length), "logsoftmax_gather_eos: null length pointer");
    return lsg_forward_dispatch(word_ins_out, dtype, select_idx, sb, sl, st, selected, require_grad, B, L, V, T, output_length,
                                target_length, nullptr, stream);
}

extern "C" int pcfgnat_logsoftmax_gather_lse(const void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl,
                                             int64_t st, void *selected, void *lse, const int64_t *output_length,
                                             const int64_t *target_length, int64_t B, int64_t L, int64_t V, int64_t T,
                                             void *stream) {
    PCFGNAT_REQUIRE(B * L == 0 || lse != nullptr, "logsoftmax_gather_lse: null lse pointer");
    PCFGNAT_REQUIRE((output_length == nullptr) == (target_length == nullptr),
                    "logsoftmax_gather_lse: output_length and target_length must be given together");
    return lsg_forward_dispatch(const_cast<void *>(word_ins_out), dtype, select_idx, sb, sl, st, selected, 0, B, L, V, T, output_length,
                                target_length, lse, stream);
}

extern "C" int pcfgnat_logsoftmax_max(const void *logits, int dtype, void *best_lprob, int64_t *best_idx, int64_t B, int64_t L,
                                      int64_t V, void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 0 && V >= 1 && V < (1LL << 31), "logsoftmax_max: bad dimensions (B=%lld L=%lld V=%lld)", (long long)B,
                    (long long)L, (long long)V);
    if (B * L == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(logits && best_lprob && best_idx, "logsoftmax_max: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case PCFGNAT_F16: return launch_ls_max<__half>(logits, best_lprob, best_idx, B * L, (int)V, s);
        case PCFGNAT_F32: return launch_ls_max<float>(logits, best_lprob, best_idx, B * L, (int)V, s);
        case PCFGNAT_F64: return launch_ls_max<double>(logits, best_lprob, best_idx, B * L, (int)V, s);
        default: return fail(PCFGNAT_EINVAL, "logsoftmax_max: unknown dtype code %d", dtype);
    }
}

static int lsg_backward_dispatch(void *buf, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl, int64_t st,
                                 const void *grad_selected, const void *lse, int64_t B, int64_t L, int64_t V, int64_t T, void *stream,
                                 const LossTask &loss = LossTask{nullptr, nullptr, nullptr, 0, 0, nullptr},
                                 const unsigned char *detach_rows = nullptr, const int64_t *pad_out_len = nullptr,
                                 int pad_rows_zeroed = 0, const float *gscale_dev = nullptr,
                                 ScaleTask also_scale = ScaleTask{nullptr, 0}) {
    int rc = check_common(buf, select_idx, grad_selected, B, L, V, T);
    if (rc != PCFGNAT_OK) return rc;
    if (B * L == 0) return PCFGNAT_OK;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case PCFGNAT_F16:
            return launch_bwd<__half>(buf, select_idx, sb, sl, st, grad_selected, B, (int)L, (int)V, (int)T, lse, loss, s, detach_rows, pad_out_len, pad_rows_zeroed, gscale_dev, also_scale);
        case PCFGNAT_F32:
            return launch_bwd<float>(buf, select_idx, sb, sl, st, grad_selected, B, (int)L, (int)V, (int)T, lse, loss, s, detach_rows, pad_out_len, pad_rows_zeroed, gscale_dev, also_scale);
        case PCFGNAT_F64:
            return launch_bwd<double>(buf, select_idx, sb, sl, st, grad_selected, B, (int)L, (int)V, (int)T, lse, loss, s, detach_rows, pad_out_len, pad_rows_zeroed, gscale_dev, also_scale);
        default:
            return fail(PCFGNAT_EINVAL, "logsoftmax_gather_backward: unknown dtype code %d", dtype);
    }
}

extern "C" int pcfgnat_logsoftmax_gather_backward(void *probs_inout, int dtype, const int64_t *select_idx, int64_t sb,
                                                  int64_t sl, int64_t st, const void *grad_selected, int64_t B, int64_t L,
                                                  int64_t V, int64_t T, void *stream) {
    return lsg_backward_dispatch(probs_inout, dtype, select_idx, sb, sl, st, grad_selected, nullptr, B, L, V, T, stream);
}

int pcfgnat::lsg_forward_eos_argmax(const void *logits, int dtype, const int64_t *targets, void *selected, int64_t *argmax,
                                    const int64_t *output_length, const int64_t *target_length, int64_t B, int64_t L, int64_t V,
                                    int64_t T, void *stream) {
    return lsg_forward_dispatch(const_cast<void *>(logits), dtype, targets, T, 0, 1, selected, 0, B, L, V, T, output_length, target_length,
                                nullptr, stream, argmax, ForceEmit{nullptr, nullptr}, 1);
}

int pcfgnat::lsg_backward_lse_with_loss(void *logits_inout, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl, int64_t st,
                                        const void *grad_selected, const void *lse, int64_t B, int64_t L, int64_t V, int64_t T,
                                        const float *S, int64_t ll_stride, const int64_t *target_length, float *loss_out,
                                        const unsigned char *keep, const int64_t *pad_output_length, int pad_rows_zeroed,
                                        const float *gscale_dev, void *stream, ScaleTask also_scale) {
    PCFGNAT_REQUIRE(B >= 1 && L >= 1 && lse && (loss_out == nullptr || (S && target_length)),
                    "logsoftmax_gather_backward: null pointer or empty batch");
    return lsg_backward_dispatch(logits_inout, dtype, select_idx, sb, sl, st, grad_selected, lse, B, L, V, T, stream,
                                 LossTask{S, target_length, loss_out, (int)B, ll_stride}, keep, pad_output_length, pad_rows_zeroed, gscale_dev,
                                 also_scale);
}

int pcfgnat::lsg_forward_lse_force(const void *logits, int dtype, const int64_t *targets, void *selected, void *lse,
                                   const int64_t *output_length, const int64_t *target_length, const unsigned char *matchmask,
                                   const unsigned char *keep, int64_t B, int64_t L, int64_t V, int64_t T, void *stream) {
    PCFGNAT_REQUIRE(B * L == 0 || (lse && output_length && target_length), "logsoftmax_gather_lse: null pointer");
    PCFGNAT_REQUIRE((matchmask == nullptr) == (keep == nullptr), "criterion_step: matchmask and keep_word_mask must be given together");
    return lsg_forward_dispatch(const_cast<void *>(logits), dtype, targets, T, 0, 1, selected, 0, B, L, V, T, output_length, target_length,
                                lse, stream, nullptr, ForceEmit{matchmask, keep}, 1);
}

extern "C" int pcfgnat_logsoftmax_gather_backward_lse(void *logits_inout, int dtype, const int64_t *select_idx, int64_t sb,
                                                      int64_t sl, int64_t st, const void *grad_selected, const void *lse, int64_t B,
                                                      int64_t L, int64_t V, int64_t T, void *stream) {
    PCFGNAT_REQUIRE(B * L == 0 || lse != nullptr, "logsoftmax_gather_backward_lse: null lse pointer");
    return lsg_backward_dispatch(logits_inout, dtype, select_idx, sb, sl, st, grad_selected, lse, B, L, V, T, stream);
}
