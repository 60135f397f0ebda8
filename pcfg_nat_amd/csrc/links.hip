// Link scorer of PCFG-NAT after its projections and its three batched products (reference
// fs_plugins/models/glat_decomposed_with_link_two_hands_tri_pcfg.py:140-201, `extract_links`), forward and backward, for
// max_left = 1 (the only value for which the reference's construction at :189-193 is defined).
//
// For parent a, left option k (k = 0: the null node 0, k = 1: node a-1) and right child c, per head h
//   z[a,k,c,h] = ( q[a,h].kl[left(a,k),h] + Zbc[h][src(a,k)][c] + Zac[h][a][c] ) / sqrt(F)
//   Zac[h][a][c] = q[a,h].kr[c,h],  Zbc[h][j][c] = kl[j,h].kr[c,h]   (batched products computed by the caller's GEMM library)
//   left(a,0) = src(a,0) = 0,  left(a,1) = max(a-1, 0),  src(a,1) = a-1 taken cyclically                       (:187-193)
//   links[a,k,c] = logsumexp_h( log_softmax_h(gate[a,:])[h] + log_softmax_{(k,c)}( z[a,:,:,h] )[k,c] )          (:168, 197-198)
// with masked entries -inf (:171-184) and unusable rows overwritten with -inf (:176-181, 199).
//
// The reference materialises z as [B,L,2L,H] (42 MB at B=40, L=128, H=8) plus several temporaries of that size, and
// autograd keeps them for the backward.  Here one workgroup per (sentence, parent) recomputes z from the two product rows
// it needs: the forward keeps only the per-head softmax normalisers, the backward emits the gradients of the two
// products and of the q.kl terms directly.  Two passes over the row in each direction (statistics, then outputs),
// nothing of size [.., 2L, H] is ever stored.
#include "common.hip.h"

namespace pcfgnat {
namespace {

constexpr int LNT = 256;
constexpr int LNW = LNT / 64;

struct RowMasks {
    bool unusable;     // no allowed left option or no allowed right child in the whole row: output -inf, gradients 0
    bool left_ok[2];   // left option k allowed
};

// right child c allowed (before the unusable-row override)
__device__ __forceinline__ bool right_allowed(const int64_t *prev, int64_t pad, const unsigned char *rtm_row,
                                              const unsigned char *main_chain, int c) {
    return !(prev[c] == pad || rtm_row[c]) && main_chain[c];
}

// Every thread of the workgroup must call this.  s_flags: two ints of LDS.
__device__ __forceinline__ RowMasks row_masks(const int64_t *prev, int64_t pad, const unsigned char *ltm_row,
                                              const unsigned char *rtm_row, const unsigned char *main_chain, int a, int L, int *s_flags,
                                              bool &right_override) {
    const int tid = threadIdx.x;
    if (tid < 2) s_flags[tid] = 0;
    __syncthreads();
    bool any_left = false, any_right = false;
    for (int j = tid; j < L; j += LNT) {
        const bool is_pad = prev[j] == pad;
        any_left |= !(is_pad || ltm_row[j]);
        any_right |= !(is_pad || rtm_row[j]) && main_chain[j];
    }
    if (any_left) s_flags[0] = 1;  // benign race: every writer stores 1
    if (any_right) s_flags[1] = 1;
    __syncthreads();
    const bool left_nouse = s_flags[0] == 0, right_nouse = s_flags[1] == 0;
    RowMasks m;
    m.unusable = left_nouse || right_nouse;
    // a row without any allowed entry on one side is computed with that side unmasked (:178-179)
    const int l1 = (a - 1 < 0) ? 0 : a - 1;
    m.left_ok[0] = left_nouse || !(prev[0] == pad || ltm_row[0]);
    m.left_ok[1] = left_nouse || !(prev[l1] == pad || ltm_row[l1]);
    right_override = right_nouse;
    return m;
}

template <int H>
__device__ __forceinline__ void block_reduce_max(float (&v)[H], float *s_red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int h = 0; h < H; h++) {
        const float w = wave_max(v[h]);
        if (lane == 0) s_red[wave * H + h] = w;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < H; h++) {
        float r = s_red[h];
        for (int w = 1; w < LNW; w++) r = fmaxf(r, s_red[w * H + h]);
        v[h] = r;
    }
    __syncthreads();
}
template <int N>
__device__ __forceinline__ void block_reduce_sum(float (&v)[N], float *s_red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int h = 0; h < N; h++) {
        const float w = wave_sum(v[h]);
        if (lane == 0) s_red[wave * N + h] = w;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < N; h++) {
        float r = s_red[h];
        for (int w = 1; w < LNW; w++) r += s_red[w * N + h];
        v[h] = r;
    }
    __syncthreads();
}

// q, kl: [B,H,L,F]; returns through s_ab[k*H+h] = q[a,h].kl[left(a,k),h] (unscaled).  Every thread must call it.
template <int H>
__device__ __forceinline__ void qkl_dots(const float *qb, const float *klb, int a, int L, int F, float *s_ab) {
    const int tid = threadIdx.x;
    if (tid < 2 * H) {
        const int k = tid / H, h = tid - k * H;
        const int left = (k == 0) ? 0 : (a - 1 < 0 ? 0 : a - 1);
        const float *qv = qb + ((size_t)h * L + a) * F, *kv = klb + ((size_t)h * L + left) * F;
        float acc = 0.f;
        for (int f = 0; f < F; f++) acc = __builtin_fmaf(qv[f], kv[f], acc);
        s_ab[tid] = acc;
    }
    __syncthreads();
}

// Forward: links [B,L,2,L], lse [B,L,H] (log-sum-exp over (k,c) of z per head), both written for every row.
template <int H>
__global__ __launch_bounds__(LNT) void links_fwd_kernel(const float *__restrict__ Zac, const float *__restrict__ Zbc,
                                                       const float *__restrict__ q, const float *__restrict__ kl,
                                                       const float *__restrict__ gate, const int64_t *__restrict__ prev_tokens,
                                                       int64_t pad, const unsigned char *__restrict__ ltm,
                                                       const unsigned char *__restrict__ rtm, const unsigned char *__restrict__ main_chain,
                                                       float *__restrict__ links, float *__restrict__ lse_out, int L, int F,
                                                       float scale) {
    __shared__ int s_flags[2];
    __shared__ float s_ab[2 * H];
    __shared__ float s_red[LNW * 2 * H];
    const int row = blockIdx.x, b = row / L, a = row - b * L, tid = threadIdx.x;
    const int64_t *prev = prev_tokens + (size_t)b * L;
    const unsigned char *ltm_row = ltm + (size_t)a * L, *rtm_row = rtm + (size_t)a * L;
    bool right_override;
    const RowMasks mk = row_masks(prev, pad, ltm_row, rtm_row, main_chain, a, L, s_flags, right_override);
    float *out = links + (size_t)row * 2 * L;
    if (mk.unusable) {  // workgroup-uniform
        for (int i = tid; i < 2 * L; i += LNT) out[i] = NEG_INF_F;
        if (tid < H) lse_out[(size_t)row * H + tid] = NEG_INF_F;
        return;
    }
    const size_t bh = (size_t)b * H;
    qkl_dots<H>(q + bh * L * F, kl + bh * L * F, a, L, F, s_ab);
    const int src1 = (a - 1 < 0) ? L - 1 : a - 1;
    // log-softmax of the gates (:168)
    float lg[H];
    {
        float mx = NEG_INF_F;
#pragma unroll
        for (int h = 0; h < H; h++) {
            lg[h] = gate[(size_t)row * H + h];
            mx = fmaxf(mx, lg[h]);
        }
        float sum = 0.f;
#pragma unroll
        for (int h = 0; h < H; h++) sum += __expf(lg[h] - mx);
        const float l = mx + __logf(sum);
#pragma unroll
        for (int h = 0; h < H; h++) lg[h] -= l;
    }
    auto z_of = [&](int k, int c, int h, bool c_ok) -> float {
        if (!mk.left_ok[k] || !c_ok) return NEG_INF_F;
        const float bc = Zbc[((bh + h) * L + (k == 0 ? 0 : src1)) * L + c];
        const float ac = Zac[((bh + h) * L + a) * L + c];
        return ((s_ab[k * H + h] * scale) + (bc * scale)) + (ac * scale);
    };
    // pass 1: per-head maximum and sum of exponentials over (k, c), online per thread
    float m[H], s[H];
#pragma unroll
    for (int h = 0; h < H; h++) {
        m[h] = NEG_INF_F;
        s[h] = 0.f;
    }
    for (int c = tid; c < L; c += LNT) {
        const bool c_ok = right_override || right_allowed(prev, pad, rtm_row, main_chain, c);
#pragma unroll
        for (int k = 0; k < 2; k++) {
#pragma unroll
            for (int h = 0; h < H; h++) {
                const float z = z_of(k, c, h, c_ok);
                if (z > m[h]) {
                    s[h] = s[h] * __expf(m[h] - z) + 1.f;  // m = -inf: 0 * 0 + 1
                    m[h] = z;
                } else if (z != NEG_INF_F) {
                    s[h] += __expf(z - m[h]);
                }
            }
        }
    }
    float M[H];
#pragma unroll
    for (int h = 0; h < H; h++) M[h] = m[h];
    block_reduce_max<H>(M, s_red);
#pragma unroll
    for (int h = 0; h < H; h++) s[h] = (m[h] == NEG_INF_F) ? 0.f : s[h] * __expf(m[h] - M[h]);
    block_reduce_sum<H>(s, s_red);
    float lse[H];
#pragma unroll
    for (int h = 0; h < H; h++) lse[h] = M[h] + __logf(s[h]);
    if (tid < H) {
        float v = 0.f;
#pragma unroll
        for (int h = 0; h < H; h++) v = (h == tid) ? lse[h] : v;
        lse_out[(size_t)row * H + tid] = v;
    }
    // pass 2: mix the heads
    for (int c = tid; c < L; c += LNT) {
        const bool c_ok = right_override || right_allowed(prev, pad, rtm_row, main_chain, c);
#pragma unroll
        for (int k = 0; k < 2; k++) {
            float t[H], mx = NEG_INF_F;
#pragma unroll
            for (int h = 0; h < H; h++) {
                t[h] = lg[h] + (z_of(k, c, h, c_ok) - lse[h]);
                mx = fmaxf(mx, t[h]);
            }
            float v = NEG_INF_F;
            if (mx != NEG_INF_F) {
                float sum = 0.f;
#pragma unroll
                for (int h = 0; h < H; h++) sum += __expf(t[h] - mx);
                v = mx + __logf(sum);
            }
            out[(size_t)k * L + c] = v;
        }
    }
}

// Backward.  dZac [B,H,L,L]: gradient of the q.kr products; dZbc1 [B,H,L,L]: the k = 1 part of the gradient of the kl.kr
// products, row src(a,1) written by parent a (a bijection, every row is written); dZ0 [B,H,L,L]: the k = 0 part per
// parent, to be summed over parents into row 0 of that gradient; dsab [B,H,L,2]: gradient of the q.kl terms;
// dgate [B,L,H]: gradient of the gate logits.  All pre-multiplied by 1/sqrt(F) where the forward scales.
template <int H>
__global__ __launch_bounds__(LNT) void links_bwd_kernel(const float *__restrict__ G, const float *__restrict__ links,
                                                       const float *__restrict__ lse_in, const float *__restrict__ Zac,
                                                       const float *__restrict__ Zbc, const float *__restrict__ q,
                                                       const float *__restrict__ kl, const float *__restrict__ gate,
                                                       const int64_t *__restrict__ prev_tokens, int64_t pad,
                                                       const unsigned char *__restrict__ ltm, const unsigned char *__restrict__ rtm,
                                                       const unsigned char *__restrict__ main_chain, float *__restrict__ dZac,
                                                       float *__restrict__ dZbc1, float *__restrict__ dZ0, float *__restrict__ dsab,
                                                       float *__restrict__ dgate, int L, int F, float scale) {
    __shared__ int s_flags[2];
    __shared__ float s_ab[2 * H];
    __shared__ float s_red[LNW * 2 * H];
    const int row = blockIdx.x, b = row / L, a = row - b * L, tid = threadIdx.x;
    const int64_t *prev = prev_tokens + (size_t)b * L;
    const unsigned char *ltm_row = ltm + (size_t)a * L, *rtm_row = rtm + (size_t)a * L;
    bool right_override;
    const RowMasks mk = row_masks(prev, pad, ltm_row, rtm_row, main_chain, a, L, s_flags, right_override);
    const size_t bh = (size_t)b * H;
    const int src1 = (a - 1 < 0) ? L - 1 : a - 1;
    if (mk.unusable) {  // the row was overwritten with a constant: no gradient flows (:199)
        for (int i = tid; i < H * L; i += LNT) {
            const int h = i / L, c = i - h * L;
            dZac[((bh + h) * L + a) * L + c] = 0.f;
            dZ0[((bh + h) * L + a) * L + c] = 0.f;
            dZbc1[((bh + h) * L + src1) * L + c] = 0.f;
        }
        if (tid < 2 * H) dsab[((bh + tid % H) * L + a) * 2 + tid / H] = 0.f;
        if (tid < H) dgate[(size_t)row * H + tid] = 0.f;
        return;
    }
    qkl_dots<H>(q + bh * L * F, kl + bh * L * F, a, L, F, s_ab);
    float lg[H], lse[H], gp[H];  // log gates, per-head normalisers, gate probabilities
    {
        float mx = NEG_INF_F;
#pragma unroll
        for (int h = 0; h < H; h++) {
            lg[h] = gate[(size_t)row * H + h];
            lse[h] = lse_in[(size_t)row * H + h];
            mx = fmaxf(mx, lg[h]);
        }
        float sum = 0.f;
#pragma unroll
        for (int h = 0; h < H; h++) sum += __expf(lg[h] - mx);
        const float l = mx + __logf(sum);
#pragma unroll
        for (int h = 0; h < H; h++) {
            lg[h] -= l;
            gp[h] = __expf(lg[h]);
        }
    }
    const float *Gr = G + (size_t)row * 2 * L, *Lr = links + (size_t)row * 2 * L;
    auto lp_of = [&](int k, int c, int h, bool c_ok) -> float {  // log-softmax over (k,c) of head h
        if (!mk.left_ok[k] || !c_ok) return NEG_INF_F;
        const float bc = Zbc[((bh + h) * L + (k == 0 ? 0 : src1)) * L + c];
        const float ac = Zac[((bh + h) * L + a) * L + c];
        return (((s_ab[k * H + h] * scale) + (bc * scale)) + (ac * scale)) - lse[h];
    };
    // pass 1: dg[h] = sum over (k,c) of G * w,  w = exp(log gate + lp - links): the share of head h in links[k,c]
    float dg[H];
#pragma unroll
    for (int h = 0; h < H; h++) dg[h] = 0.f;
    for (int c = tid; c < L; c += LNT) {
        const bool c_ok = right_override || right_allowed(prev, pad, rtm_row, main_chain, c);
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const float lk = Lr[(size_t)k * L + c], g = Gr[(size_t)k * L + c];
            if (lk == NEG_INF_F) continue;  // masked entry: a constant, no gradient
#pragma unroll
            for (int h = 0; h < H; h++) {
                const float lp = lp_of(k, c, h, c_ok);
                if (lp != NEG_INF_F) dg[h] += g * __expf((lg[h] + lp) - lk);
            }
        }
    }
    block_reduce_sum<H>(dg, s_red);
    // gradient of the gate logits through their log-softmax
    if (tid < H) {
        float tot = 0.f, mine = 0.f, gpm = 0.f;
#pragma unroll
        for (int h = 0; h < H; h++) {
            tot += dg[h];
            mine = (h == tid) ? dg[h] : mine;
            gpm = (h == tid) ? gp[h] : gpm;
        }
        dgate[(size_t)row * H + tid] = mine - gpm * tot;
    }
    // pass 2: dz = G*w - softmax * dg[h]
    float ds[2 * H];
#pragma unroll
    for (int i = 0; i < 2 * H; i++) ds[i] = 0.f;
    for (int c = tid; c < L; c += LNT) {
        const bool c_ok = right_override || right_allowed(prev, pad, rtm_row, main_chain, c);
        const float lk0 = Lr[c], lk1 = Lr[(size_t)L + c], g0 = Gr[c], g1 = Gr[(size_t)L + c];
#pragma unroll
        for (int h = 0; h < H; h++) {
            float dz[2];
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const float lp = lp_of(k, c, h, c_ok);
                const float lk = k ? lk1 : lk0, g = k ? g1 : g0;
                float v = 0.f;
                if (lp != NEG_INF_F) {
                    const float w = (lk == NEG_INF_F) ? 0.f : g * __expf((lg[h] + lp) - lk);
                    v = (w - __expf(lp) * dg[h]) * scale;
                }
                dz[k] = v;
                ds[k * H + h] += v;
            }
            dZac[((bh + h) * L + a) * L + c] = dz[0] + dz[1];
            dZ0[((bh + h) * L + a) * L + c] = dz[0];
            dZbc1[((bh + h) * L + src1) * L + c] = dz[1];
        }
    }
    block_reduce_sum<2 * H>(ds, s_red);
    if (tid < 2 * H) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < 2 * H; i++) v = (i == tid) ? ds[i] : v;
        dsab[((bh + tid % H) * L + a) * 2 + tid / H] = v;
    }
}

int check_links_args(const char *who, int64_t B, int64_t L, int64_t H, int64_t F) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 2 && F >= 1, "%s: bad dimensions (B=%lld L=%lld F=%lld)", who, (long long)B, (long long)L, (long long)F);
    PCFGNAT_REQUIRE(L <= 8192, "%s: graph too large (L <= 8192)", who);
    if (!(H == 1 || H == 2 || H == 4 || H == 8 || H == 16))
        return fail(PCFGNAT_EUNSUPPORTED, "%s: %lld attention heads (1, 2, 4, 8 and 16 are built)", who, (long long)H);
    return PCFGNAT_OK;
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

extern "C" int pcfgnat_extract_links_forward(const float *Zac, const float *Zbc, const float *q, const float *kl, const float *gate_logits,
                                             const int64_t *prev_output_tokens, int64_t pad_index, const unsigned char *left_tree_mask,
                                             const unsigned char *right_tree_mask, const unsigned char *main_chain, float *links,
                                             float *head_lse, int64_t B, int64_t L, int64_t H, int64_t F, void *stream) {
    int rc = check_links_args("extract_links_forward", B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(Zac && Zbc && q && kl && gate_logits && prev_output_tokens && left_tree_mask && right_tree_mask && main_chain &&
                        links && head_lse,
                    "extract_links_forward: null pointer");
    const float scale = 1.0f / sqrtf((float)F);
    hipStream_t s = (hipStream_t)stream;
#define PCFGNAT_LINKS_FWD(h)                                                                                                          \
    case h:                                                                                                                           \
        hipLaunchKernelGGL((links_fwd_kernel<h>), dim3((unsigned)(B * L)), dim3(LNT), 0, s, Zac, Zbc, q, kl, gate_logits,               \
                           prev_output_tokens, pad_index, left_tree_mask, right_tree_mask, main_chain, links, head_lse, (int)L, (int)F, \
                           scale);                                                                                                    \
        break
    switch (H) {
        PCFGNAT_LINKS_FWD(1);
        PCFGNAT_LINKS_FWD(2);
        PCFGNAT_LINKS_FWD(4);
        PCFGNAT_LINKS_FWD(8);
        PCFGNAT_LINKS_FWD(16);
    }
#undef PCFGNAT_LINKS_FWD
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_extract_links_backward(const float *grad_links, const float *links, const float *head_lse, const float *Zac,
                                              const float *Zbc, const float *q, const float *kl, const float *gate_logits,
                                              const int64_t *prev_output_tokens, int64_t pad_index, const unsigned char *left_tree_mask,
                                              const unsigned char *right_tree_mask, const unsigned char *main_chain, float *dZac,
                                              float *dZbc1, float *dZ0, float *dsab, float *dgate, int64_t B, int64_t L, int64_t H,
                                              int64_t F, void *stream) {
    int rc = check_links_args("extract_links_backward", B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(grad_links && links && head_lse && Zac && Zbc && q && kl && gate_logits && prev_output_tokens && left_tree_mask &&
                        right_tree_mask && main_chain && dZac && dZbc1 && dZ0 && dsab && dgate,
                    "extract_links_backward: null pointer");
    const float scale = 1.0f / sqrtf((float)F);
    hipStream_t s = (hipStream_t)stream;
#define PCFGNAT_LINKS_BWD(h)                                                                                                            \
    case h:                                                                                                                             \
        hipLaunchKernelGGL((links_bwd_kernel<h>), dim3((unsigned)(B * L)), dim3(LNT), 0, s, grad_links, links, head_lse, Zac, Zbc, q, kl, \
                           gate_logits, prev_output_tokens, pad_index, left_tree_mask, right_tree_mask, main_chain, dZac, dZbc1, dZ0,   \
                           dsab, dgate, (int)L, (int)F, scale);                                                                         \
        break
    switch (H) {
        PCFGNAT_LINKS_BWD(1);
        PCFGNAT_LINKS_BWD(2);
        PCFGNAT_LINKS_BWD(4);
        PCFGNAT_LINKS_BWD(8);
        PCFGNAT_LINKS_BWD(16);
    }
#undef PCFGNAT_LINKS_BWD
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
