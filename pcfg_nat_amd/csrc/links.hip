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
// products and of the q.kl terms directly.  One wave64 per (sentence, parent) row, lanes strided over the right children,
// two passes over the row in each direction (statistics, then outputs) with the scores held in registers in between for
// graphs of up to 256 nodes; no workgroup barrier, nothing of size [.., 2L, H] is ever stored.
#include "common.hip.h"

namespace pcfgnat {
namespace {

constexpr int LNT = 256;          // threads per workgroup
constexpr int ROWS = LNT / 64;    // one wave64 per (sentence, parent) row: no workgroup barriers anywhere

struct RowMasks {
    bool unusable;        // no allowed left option or no allowed right child in the whole row: output -inf, gradients 0
    bool left_ok[2];      // left option k allowed
    bool right_override;  // the row has no allowed right child: computed with the right side unmasked (:179)
};

// right child c allowed (before the unusable-row override)
__device__ __forceinline__ bool right_allowed(const int64_t *prev, int64_t pad, const unsigned char *rtm_row,
                                              const unsigned char *main_chain, int c) {
    return !(prev[c] == pad || rtm_row[c]) && main_chain[c];
}

// Called by all lanes of the wave that owns the row.
__device__ __forceinline__ RowMasks row_masks(const int64_t *prev, int64_t pad, const unsigned char *ltm_row,
                                              const unsigned char *rtm_row, const unsigned char *main_chain, int a, int L) {
    const int lane = threadIdx.x & 63;
    bool any_left = false, any_right = false;
    for (int j = lane; j < L; j += 64) {
        const bool is_pad = prev[j] == pad;
        any_left |= !(is_pad || ltm_row[j]);
        any_right |= !(is_pad || rtm_row[j]) && main_chain[j];
    }
    const bool left_nouse = !__any(any_left), right_nouse = !__any(any_right);
    RowMasks m;
    m.unusable = left_nouse || right_nouse;
    // a row without any allowed entry on one side is computed with that side unmasked (:178-179)
    const int l1 = (a - 1 < 0) ? 0 : a - 1;
    m.left_ok[0] = left_nouse || !(prev[0] == pad || ltm_row[0]);
    m.left_ok[1] = left_nouse || !(prev[l1] == pad || ltm_row[l1]);
    m.right_override = right_nouse;
    return m;
}

// qb, klb: the query / left-key rows of one sentence, head h at offset h*qh, row l at l*F;
// sab[k*H+h] = q[a,h].kl[left(a,k),h] (unscaled), the same in every lane.
template <int H>
__device__ __forceinline__ void qkl_dots(const float *qb, const float *klb, size_t qh, int a, int F, float (&sab)[2 * H]) {
    const int lane = threadIdx.x & 63;
    const int l1 = (a - 1 < 0) ? 0 : a - 1;
#pragma unroll
    for (int d = 0; d < 2 * H; d++) {
        const int k = d / H, h = d - k * H;
        const float *qv = qb + h * qh + (size_t)a * F, *kv = klb + h * qh + (size_t)(k == 0 ? 0 : l1) * F;
        float acc = 0.f;
        for (int f = lane; f < F; f += 64) acc = __builtin_fmaf(qv[f], kv[f], acc);
        sab[d] = wave_sum(acc);
    }
}

template <int H>
__device__ __forceinline__ void log_gates(const float *gate_row, float (&lg)[H]) {
    float mx = NEG_INF_F;
#pragma unroll
    for (int h = 0; h < H; h++) {
        lg[h] = gate_row[h];
        mx = fmaxf(mx, lg[h]);
    }
    float sum = 0.f;
#pragma unroll
    for (int h = 0; h < H; h++) sum += __expf(lg[h] - mx);
    const float l = mx + __logf(sum);
#pragma unroll
    for (int h = 0; h < H; h++) lg[h] -= l;
}

// The scaled scores of one right child c for both left options and all heads, -inf where masked.
template <int H>
struct RowScores {
    const float *Zac_row, *Zbc_row0, *Zbc_row1;  // row a of Zac, rows 0 and src(a,1) of Zbc, head 0; head stride = L*L
    size_t head_stride;
    float sab[2 * H];
    float scale;
    bool left_ok[2];
    __device__ __forceinline__ void at(int c, bool c_ok, float (&z)[2][H]) const {
#pragma unroll
        for (int h = 0; h < H; h++) {
            const float ac = Zac_row[h * head_stride + c] * scale;
            const float b0 = Zbc_row0[h * head_stride + c] * scale, b1 = Zbc_row1[h * head_stride + c] * scale;
            z[0][h] = (left_ok[0] && c_ok) ? ((sab[h] * scale) + b0) + ac : NEG_INF_F;
            z[1][h] = (left_ok[1] && c_ok) ? ((sab[H + h] * scale) + b1) + ac : NEG_INF_F;
        }
    }
};

// Forward: links [B,L,2,L], lse [B,L,H] (log-sum-exp over (k,c) of z per head), both written for every row.
// CPL > 0: the scores of up to CPL columns per lane stay in registers between the two passes (L <= 64*CPL);
// CPL = 0: they are recomputed.
template <int H, int CPL>
__global__ __launch_bounds__(LNT) void links_fwd_kernel(const float *__restrict__ Zac, const float *__restrict__ Zbc,
                                                       const float *__restrict__ q, const float *__restrict__ kl,
                                                       const float *__restrict__ gate, const int64_t *__restrict__ prev_tokens,
                                                       int64_t pad, const unsigned char *__restrict__ ltm,
                                                       const unsigned char *__restrict__ rtm, const unsigned char *__restrict__ main_chain,
                                                       float *__restrict__ links, float *__restrict__ lse_out, int rows, int L, int F,
                                                       float scale, size_t zh, size_t qh) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * ROWS + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int b = row / L, a = row - b * L;
    const int64_t *prev = prev_tokens + (size_t)b * L;
    const unsigned char *ltm_row = ltm + (size_t)a * L, *rtm_row = rtm + (size_t)a * L;
    const RowMasks mk = row_masks(prev, pad, ltm_row, rtm_row, main_chain, a, L);
    float *out = links + (size_t)row * 2 * L;
    if (mk.unusable) {  // wave-uniform
        for (int i = lane; i < 2 * L; i += 64) out[i] = NEG_INF_F;
        if (lane < H) lse_out[(size_t)row * H + lane] = NEG_INF_F;
        return;
    }
    const size_t bh = (size_t)b * H;
    const int src1 = (a - 1 < 0) ? L - 1 : a - 1;
    RowScores<H> sc;
    sc.head_stride = zh;
    sc.Zac_row = Zac + bh * zh + (size_t)a * L;
    sc.Zbc_row0 = Zbc + bh * zh;
    sc.Zbc_row1 = Zbc + bh * zh + (size_t)src1 * L;
    sc.scale = scale;
    sc.left_ok[0] = mk.left_ok[0];
    sc.left_ok[1] = mk.left_ok[1];
    qkl_dots<H>(q + bh * qh, kl + bh * qh, qh, a, F, sc.sab);
    float lg[H];
    log_gates<H>(gate + (size_t)row * H, lg);

    // pass 1: per-head maximum and sum of exponentials over (k, c), online per lane
    float m[H], s[H];
#pragma unroll
    for (int h = 0; h < H; h++) {
        m[h] = NEG_INF_F;
        s[h] = 0.f;
    }
    float zc[CPL > 0 ? CPL : 1][2][H];
    auto fold = [&](const float (&z)[2][H]) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
#pragma unroll
            for (int h = 0; h < H; h++) {
                const float v = z[k][h];
                if (v > m[h]) {
                    s[h] = s[h] * __expf(m[h] - v) + 1.f;  // m = -inf: 0 * 0 + 1
                    m[h] = v;
                } else if (v != NEG_INF_F) {
                    s[h] += __expf(v - m[h]);
                }
            }
        }
    };
    if (CPL > 0) {
#pragma unroll
        for (int i = 0; i < (CPL > 0 ? CPL : 1); i++) {
            const int c = lane + 64 * i;
            const bool in = c < L;
            const int cc = in ? c : 0;
            sc.at(cc, in && (mk.right_override || right_allowed(prev, pad, rtm_row, main_chain, cc)), zc[i]);
            fold(zc[i]);
        }
    } else {
        for (int c = lane; c < L; c += 64) {
            float z[2][H];
            sc.at(c, mk.right_override || right_allowed(prev, pad, rtm_row, main_chain, c), z);
            fold(z);
        }
    }
    float lse[H];
#pragma unroll
    for (int h = 0; h < H; h++) {
        const float M = wave_max(m[h]);
        const float part = (m[h] == NEG_INF_F) ? 0.f : s[h] * __expf(m[h] - M);
        lse[h] = M + __logf(wave_sum(part));
    }
    if (lane < H) {
        float v = 0.f;
#pragma unroll
        for (int h = 0; h < H; h++) v = (h == lane) ? lse[h] : v;
        lse_out[(size_t)row * H + lane] = v;
    }
    // pass 2: mix the heads
    auto emit = [&](int c, const float (&z)[2][H]) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
            float t[H], mx = NEG_INF_F;
#pragma unroll
            for (int h = 0; h < H; h++) {
                t[h] = lg[h] + (z[k][h] - lse[h]);
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
    };
    if (CPL > 0) {
#pragma unroll
        for (int i = 0; i < (CPL > 0 ? CPL : 1); i++) {
            const int c = lane + 64 * i;
            if (c < L) emit(c, zc[i]);
        }
    } else {
        for (int c = lane; c < L; c += 64) {
            float z[2][H];
            sc.at(c, mk.right_override || right_allowed(prev, pad, rtm_row, main_chain, c), z);
            emit(c, z);
        }
    }
}

// Backward.  dZac [B,H,L,L]: gradient of the q.kr products; dZbc1 [B,H,L,L]: the k = 1 part of the gradient of the kl.kr
// products, row src(a,1) written by parent a (a bijection, every row is written); dZ0 [B,H,L,L]: the k = 0 part per
// parent, to be summed over parents into row 0 of that gradient; dsab [B,H,L,2]: gradient of the q.kl terms;
// dgate [B,L,H]: gradient of the gate logits.  All pre-multiplied by 1/sqrt(F) where the forward scales.
template <int H, int CPL>
__global__ __launch_bounds__(LNT) void links_bwd_kernel(const float *__restrict__ G, const float *__restrict__ links,
                                                       const float *__restrict__ lse_in, const float *__restrict__ Zac,
                                                       const float *__restrict__ Zbc, const float *__restrict__ q,
                                                       const float *__restrict__ kl, const float *__restrict__ gate,
                                                       const int64_t *__restrict__ prev_tokens, int64_t pad,
                                                       const unsigned char *__restrict__ ltm, const unsigned char *__restrict__ rtm,
                                                       const unsigned char *__restrict__ main_chain, float *__restrict__ dZac,
                                                       float *__restrict__ dZbc1, float *__restrict__ dZ0, float *__restrict__ dsab,
                                                       float *__restrict__ dgate, int rows, int L, int F, float scale, size_t zh,
                                                       size_t qh) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * ROWS + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int b = row / L, a = row - b * L;
    const int64_t *prev = prev_tokens + (size_t)b * L;
    const unsigned char *ltm_row = ltm + (size_t)a * L, *rtm_row = rtm + (size_t)a * L;
    const RowMasks mk = row_masks(prev, pad, ltm_row, rtm_row, main_chain, a, L);
    const size_t bh = (size_t)b * H;
    const int src1 = (a - 1 < 0) ? L - 1 : a - 1;
    const size_t hs = (size_t)L * L;  // head stride of dZ0; dZac / dZbc1 share the stride zh of the products
    float *dZac_row = dZac + bh * zh + (size_t)a * L, *dZ0_row = dZ0 + (bh * L + a) * L, *dZbc1_row = dZbc1 + bh * zh + (size_t)src1 * L;
    if (mk.unusable) {  // the row was overwritten with a constant: no gradient flows (:199)
        for (int i = lane; i < H * L; i += 64) {
            const int h = i / L, c = i - h * L;
            dZac_row[h * zh + c] = 0.f;
            dZ0_row[h * hs + c] = 0.f;
            dZbc1_row[h * zh + c] = 0.f;
        }
        if (lane < 2 * H) dsab[((bh + lane % H) * L + a) * 2 + lane / H] = 0.f;
        if (lane < H) dgate[(size_t)row * H + lane] = 0.f;
        return;
    }
    RowScores<H> sc;
    sc.head_stride = zh;
    sc.Zac_row = Zac + bh * zh + (size_t)a * L;
    sc.Zbc_row0 = Zbc + bh * zh;
    sc.Zbc_row1 = Zbc + bh * zh + (size_t)src1 * L;
    sc.scale = scale;
    sc.left_ok[0] = mk.left_ok[0];
    sc.left_ok[1] = mk.left_ok[1];
    qkl_dots<H>(q + bh * qh, kl + bh * qh, qh, a, F, sc.sab);
    float lg[H], lse[H];
    log_gates<H>(gate + (size_t)row * H, lg);
#pragma unroll
    for (int h = 0; h < H; h++) lse[h] = lse_in[(size_t)row * H + h];
    const float *Gr = G + (size_t)row * 2 * L, *Lr = links + (size_t)row * 2 * L;

    // pass 1: dg[h] = sum over (k,c) of G * w,  w = exp(log gate + lp - links): the share of head h in links[k,c]
    // (lp = z - lse[h]: log-softmax over (k,c) of head h).  wgt[k][h] = G * w is kept per cached column.
    float dg[H];
#pragma unroll
    for (int h = 0; h < H; h++) dg[h] = 0.f;
    float zc[CPL > 0 ? CPL : 1][2][H];
    auto shares = [&](int c, const float (&z)[2][H], float (&gw)[2][H]) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const float lk = Lr[(size_t)k * L + c], g = Gr[(size_t)k * L + c];
#pragma unroll
            for (int h = 0; h < H; h++) {
                const float lp = z[k][h] - lse[h];
                // masked entries (links = -inf) are constants: no gradient
                gw[k][h] = (lk == NEG_INF_F || z[k][h] == NEG_INF_F) ? 0.f : g * __expf((lg[h] + lp) - lk);
            }
        }
    };
    if (CPL > 0) {
#pragma unroll
        for (int i = 0; i < (CPL > 0 ? CPL : 1); i++) {
            const int c = lane + 64 * i;
            const bool in = c < L;
            const int cc = in ? c : 0;
            sc.at(cc, in && (mk.right_override || right_allowed(prev, pad, rtm_row, main_chain, cc)), zc[i]);
            float gw[2][H];
            shares(cc, zc[i], gw);
#pragma unroll
            for (int h = 0; h < H; h++) dg[h] += gw[0][h] + gw[1][h];
        }
    } else {
        for (int c = lane; c < L; c += 64) {
            float z[2][H], gw[2][H];
            sc.at(c, mk.right_override || right_allowed(prev, pad, rtm_row, main_chain, c), z);
            shares(c, z, gw);
#pragma unroll
            for (int h = 0; h < H; h++) dg[h] += gw[0][h] + gw[1][h];
        }
    }
#pragma unroll
    for (int h = 0; h < H; h++) dg[h] = wave_sum(dg[h]);
    // gradient of the gate logits through their log-softmax
    if (lane < H) {
        float tot = 0.f, mine = 0.f, lgm = 0.f;
#pragma unroll
        for (int h = 0; h < H; h++) {
            tot += dg[h];
            mine = (h == lane) ? dg[h] : mine;
            lgm = (h == lane) ? lg[h] : lgm;
        }
        dgate[(size_t)row * H + lane] = mine - __expf(lgm) * tot;
    }
    // pass 2: dz = G*w - softmax * dg[h]
    float ds[2 * H];
#pragma unroll
    for (int i = 0; i < 2 * H; i++) ds[i] = 0.f;
    auto emit = [&](int c, const float (&z)[2][H]) {
        float gw[2][H];
        shares(c, z, gw);
#pragma unroll
        for (int h = 0; h < H; h++) {
            float dz[2];
#pragma unroll
            for (int k = 0; k < 2; k++) {
                dz[k] = (z[k][h] == NEG_INF_F) ? 0.f : (gw[k][h] - __expf(z[k][h] - lse[h]) * dg[h]) * scale;
                ds[k * H + h] += dz[k];
            }
            dZac_row[h * zh + c] = dz[0] + dz[1];
            dZ0_row[h * hs + c] = dz[0];
            dZbc1_row[h * zh + c] = dz[1];
        }
    };
    if (CPL > 0) {
#pragma unroll
        for (int i = 0; i < (CPL > 0 ? CPL : 1); i++) {
            const int c = lane + 64 * i;
            if (c < L) emit(c, zc[i]);
        }
    } else {
        for (int c = lane; c < L; c += 64) {
            float z[2][H];
            sc.at(c, mk.right_override || right_allowed(prev, pad, rtm_row, main_chain, c), z);
            emit(c, z);
        }
    }
#pragma unroll
    for (int i = 0; i < 2 * H; i++) ds[i] = wave_sum(ds[i]);
    if (lane < 2 * H) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < 2 * H; i++) v = (i == lane) ? ds[i] : v;
        dsab[((bh + lane % H) * L + a) * 2 + lane / H] = v;
    }
}

// Packs the three projections [B,L,H,F] (any of the supported dtypes) into the float32 operands of the two batched
// products: A [B,H,2L,F] (query rows, then left-key rows) and Kr [B,H,L,F].
template <typename T>
__global__ __launch_bounds__(256) void links_pack_kernel(const T *__restrict__ q, const T *__restrict__ kl, const T *__restrict__ kr,
                                                        float *__restrict__ A, float *__restrict__ Kr, int B, int L, int H, int F) {
    const size_t n = (size_t)B * L * H * F;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const int f = (int)(i % F);
        size_t r = i / F;
        const int h = (int)(r % H);
        r /= H;
        const int l = (int)(r % L), b = (int)(r / L);
        const size_t bh = (size_t)b * H + h;
        A[(bh * 2 * L + l) * F + f] = (float)q[i];
        A[(bh * 2 * L + L + l) * F + f] = (float)kl[i];
        Kr[(bh * L + l) * F + f] = (float)kr[i];
    }
}

// dZ[b,h,L+0,c] += sum over parents a of dZ0[b,h,a,c]: every parent's null left child is node 0.  One block per
// (b*H + h, tile of 64 columns): four groups of 64 threads sum a quarter of the parents each.
__global__ __launch_bounds__(256) void links_colsum_kernel(const float *__restrict__ dZ0, float *__restrict__ dZ, int L) {
    __shared__ float s_part[4][64];
    const size_t bh = blockIdx.x;
    const int c = blockIdx.y * 64 + (threadIdx.x & 63), g = threadIdx.x >> 6;
    float acc = 0.f;
    if (c < L) {
        const float *col = dZ0 + bh * L * L + c;
#pragma unroll 8
        for (int a = g; a < L; a += 4) acc += col[(size_t)a * L];
    }
    s_part[g][threadIdx.x & 63] = acc;
    __syncthreads();
    if (g == 0 && c < L) dZ[(bh * 2 * L + L) * L + c] += (s_part[0][threadIdx.x] + s_part[1][threadIdx.x]) + (s_part[2][threadIdx.x] + s_part[3][threadIdx.x]);
}

// Gradients of the projections from the gradients of the packed operands: dA [B,H,2L,F], dKr [B,H,L,F], plus the q.kl
// terms (dsab [B,H,L,2]: with kl[0] and with kl[max(a-1,0)]).  grid (B*H, parts): each block handles a range of rows of
// one (b,h); threads run over (row, f) with f fastest.  Dynamic LDS: F floats.
template <typename T>
__global__ __launch_bounds__(256) void links_unpack_kernel(const float *__restrict__ dA, const float *__restrict__ dKr,
                                                          const float *__restrict__ dsab, const float *__restrict__ A,
                                                          T *__restrict__ dq, T *__restrict__ dkl, T *__restrict__ dkr, int L, int H,
                                                          int F) {
    extern __shared__ float s_null[];  // [F]: sum over parents a of dsab[a][0] * q[a]  (every parent's null option)
    const size_t bh = blockIdx.x;
    const int b = (int)(bh / H), h = (int)(bh % H);
    const int rows_per = (L + gridDim.y - 1) / gridDim.y;
    const int l_begin = blockIdx.y * rows_per, l_end = min(L, l_begin + rows_per);
    const float *Aq = A + bh * 2 * L * F, *Akl = Aq + (size_t)L * F;
    const float *ds = dsab + bh * L * 2;
    const int tid = threadIdx.x;
    if (l_begin == 0) {
        for (int f = tid; f < F; f += 256) {
            float acc = 0.f;
#pragma unroll 4
            for (int a = 0; a < L; a++) acc += ds[a * 2 + 0] * Aq[(size_t)a * F + f];
            s_null[f] = acc + ds[1] * Aq[f];  // plus parent 0's clamped left index
        }
        __syncthreads();
    }
    const int n = (l_end - l_begin) * F;
    for (int i = tid; i < n; i += 256) {
        const int l = l_begin + i / F, f = i % F;
        const float d0 = ds[l * 2 + 0], d1 = ds[l * 2 + 1];
        const int lp = (l - 1 < 0) ? 0 : l - 1;
        const size_t o = (((size_t)b * L + l) * H + h) * F + f;
        dq[o] = (T)(dA[(bh * 2 * L + l) * F + f] + d0 * Akl[f] + d1 * Akl[(size_t)lp * F + f]);
        float g = dA[(bh * 2 * L + L + l) * F + f];
        if (l + 1 < L) g += ds[(l + 1) * 2 + 1] * Aq[(size_t)(l + 1) * F + f];  // parent l+1 took kl[l] as its left term
        if (l == 0) g += s_null[f];
        dkl[o] = (T)g;
        dkr[o] = (T)dKr[(bh * L + l) * F + f];
    }
}

// columns per lane kept in registers: as many as fit in 64 floats of scores per lane
int cached_columns(int64_t L, int64_t H) {
    if (L <= 128 && 2 * 2 * H <= 64) return 2;
    if (L <= 256 && 4 * 2 * H <= 64) return 4;
    return 0;
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

namespace {
template <typename T>
int launch_pack(const void *q, const void *kl, const void *kr, float *A, float *Kr, int64_t B, int64_t L, int64_t H, int64_t F,
                hipStream_t s) {
    const size_t n = (size_t)B * L * H * F;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65535 * 8 ? (n + 255) / 256 : 65535 * 8);
    hipLaunchKernelGGL((links_pack_kernel<T>), dim3(grid), dim3(256), 0, s, (const T *)q, (const T *)kl, (const T *)kr, A, Kr, (int)B, (int)L,
                       (int)H, (int)F);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
template <typename T>
int launch_unpack(const float *dA, const float *dKr, const float *dsab, const float *A, void *dq, void *dkl, void *dkr, int64_t B,
                  int64_t L, int64_t H, int64_t F, hipStream_t s) {
    const unsigned parts = (unsigned)(L >= 64 ? 8 : 1);
    hipLaunchKernelGGL((links_unpack_kernel<T>), dim3((unsigned)(B * H), parts), dim3(256), (size_t)F * sizeof(float), s, dA, dKr, dsab, A,
                       (T *)dq, (T *)dkl, (T *)dkr, (int)L, (int)H, (int)F);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
}  // namespace

extern "C" int pcfgnat_extract_links_pack(const void *query_chunks, const void *key_chunks_left, const void *key_chunks_right, int dtype,
                                          float *A, float *Kr, int64_t B, int64_t L, int64_t H, int64_t F, void *stream) {
    int rc = check_links_args("extract_links_pack", B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(query_chunks && key_chunks_left && key_chunks_right && A && Kr, "extract_links_pack: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case PCFGNAT_F16: return launch_pack<__half>(query_chunks, key_chunks_left, key_chunks_right, A, Kr, B, L, H, F, s);
        case PCFGNAT_F32: return launch_pack<float>(query_chunks, key_chunks_left, key_chunks_right, A, Kr, B, L, H, F, s);
        case PCFGNAT_F64: return launch_pack<double>(query_chunks, key_chunks_left, key_chunks_right, A, Kr, B, L, H, F, s);
        default: return fail(PCFGNAT_EINVAL, "extract_links_pack: unknown dtype code %d", dtype);
    }
}

extern "C" int pcfgnat_extract_links_forward(const float *Z, const float *A, const float *gate_logits, const int64_t *prev_output_tokens,
                                             int64_t pad_index, const unsigned char *left_tree_mask, const unsigned char *right_tree_mask,
                                             const unsigned char *main_chain, float *links, float *head_lse, int64_t B, int64_t L,
                                             int64_t H, int64_t F, void *stream) {
    int rc = check_links_args("extract_links_forward", B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(Z && A && gate_logits && prev_output_tokens && left_tree_mask && right_tree_mask && main_chain && links && head_lse,
                    "extract_links_forward: null pointer");
    const float scale = 1.0f / sqrtf((float)F);
    hipStream_t s = (hipStream_t)stream;
    const float *Zac = Z, *Zbc = Z + (size_t)L * L, *q = A, *kl = A + (size_t)L * F;
    const size_t zh = (size_t)2 * L * L, qh = (size_t)2 * L * F;
    const int rows = (int)(B * L), cpl = cached_columns(L, H);
    const dim3 grid((unsigned)((rows + ROWS - 1) / ROWS));
#define PCFGNAT_LINKS_FWD_C(h, c)                                                                                                      \
    hipLaunchKernelGGL((links_fwd_kernel<h, c>), grid, dim3(LNT), 0, s, Zac, Zbc, q, kl, gate_logits, prev_output_tokens, pad_index,     \
                       left_tree_mask, right_tree_mask, main_chain, links, head_lse, rows, (int)L, (int)F, scale, zh, qh)
#define PCFGNAT_LINKS_FWD(h)                                         \
    case h:                                                          \
        if (cpl == 2) PCFGNAT_LINKS_FWD_C(h, 2);                     \
        else if (cpl == 4) PCFGNAT_LINKS_FWD_C(h, (h <= 8 ? 4 : 0)); \
        else PCFGNAT_LINKS_FWD_C(h, 0);                              \
        break
    switch (H) {
        PCFGNAT_LINKS_FWD(1);
        PCFGNAT_LINKS_FWD(2);
        PCFGNAT_LINKS_FWD(4);
        PCFGNAT_LINKS_FWD(8);
        PCFGNAT_LINKS_FWD(16);
    }
#undef PCFGNAT_LINKS_FWD_C
#undef PCFGNAT_LINKS_FWD
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_extract_links_backward(const float *grad_links, const float *links, const float *head_lse, const float *Z,
                                              const float *A, const float *gate_logits, const int64_t *prev_output_tokens,
                                              int64_t pad_index, const unsigned char *left_tree_mask,
                                              const unsigned char *right_tree_mask, const unsigned char *main_chain, float *dZ, float *dZ0,
                                              float *dsab, float *dgate, int64_t B, int64_t L, int64_t H, int64_t F, void *stream) {
    int rc = check_links_args("extract_links_backward", B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(grad_links && links && head_lse && Z && A && gate_logits && prev_output_tokens && left_tree_mask && right_tree_mask &&
                        main_chain && dZ && dZ0 && dsab && dgate,
                    "extract_links_backward: null pointer");
    const float scale = 1.0f / sqrtf((float)F);
    hipStream_t s = (hipStream_t)stream;
    const float *Zac = Z, *Zbc = Z + (size_t)L * L, *q = A, *kl = A + (size_t)L * F;
    float *dZac = dZ, *dZbc1 = dZ + (size_t)L * L;
    const size_t zh = (size_t)2 * L * L, qh = (size_t)2 * L * F;
    const int rows = (int)(B * L), cpl = cached_columns(L, H);
    const dim3 grid((unsigned)((rows + ROWS - 1) / ROWS));
#define PCFGNAT_LINKS_BWD_C(h, c)                                                                                                        \
    hipLaunchKernelGGL((links_bwd_kernel<h, c>), grid, dim3(LNT), 0, s, grad_links, links, head_lse, Zac, Zbc, q, kl, gate_logits,         \
                       prev_output_tokens, pad_index, left_tree_mask, right_tree_mask, main_chain, dZac, dZbc1, dZ0, dsab, dgate, rows,   \
                       (int)L, (int)F, scale, zh, qh)
#define PCFGNAT_LINKS_BWD(h)                                         \
    case h:                                                          \
        if (cpl == 2) PCFGNAT_LINKS_BWD_C(h, 2);                     \
        else if (cpl == 4) PCFGNAT_LINKS_BWD_C(h, (h <= 8 ? 4 : 0)); \
        else PCFGNAT_LINKS_BWD_C(h, 0);                              \
        break
    switch (H) {
        PCFGNAT_LINKS_BWD(1);
        PCFGNAT_LINKS_BWD(2);
        PCFGNAT_LINKS_BWD(4);
        PCFGNAT_LINKS_BWD(8);
        PCFGNAT_LINKS_BWD(16);
    }
#undef PCFGNAT_LINKS_BWD_C
#undef PCFGNAT_LINKS_BWD
    PCFGNAT_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(links_colsum_kernel, dim3((unsigned)(B * H), (unsigned)((L + 63) / 64)), dim3(256), 0, s, dZ0, dZ, (int)L);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_extract_links_unpack(const float *dA, const float *dKr, const float *dsab, const float *A, int dtype, void *dq,
                                            void *dkl, void *dkr, int64_t B, int64_t L, int64_t H, int64_t F, void *stream) {
    int rc = check_links_args("extract_links_unpack", B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(dA && dKr && dsab && A && dq && dkl && dkr, "extract_links_unpack: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case PCFGNAT_F16: return launch_unpack<__half>(dA, dKr, dsab, A, dq, dkl, dkr, B, L, H, F, s);
        case PCFGNAT_F32: return launch_unpack<float>(dA, dKr, dsab, A, dq, dkl, dkr, B, L, H, F, s);
        case PCFGNAT_F64: return launch_unpack<double>(dA, dKr, dsab, A, dq, dkl, dkr, B, L, H, F, s);
        default: return fail(PCFGNAT_EINVAL, "extract_links_unpack: unknown dtype code %d", dtype);
    }
}
