// Link scorer of PCFG-NAT (reference fs_plugins/models/glat_decomposed_with_link_two_hands_tri_pcfg.py:140-201,
// `extract_links`, after its four projections) with its three batched products on the matrix cores inside the kernels:
// one launch forward, nothing of size [B,L,2L,H] or [B,H,2L,L] stored in either direction.  max_left = 1.
//
// For parent a, left option k (k = 0: the null node 0, k = 1: node a-1) and right child c, per head h
//   z[a,k,c,h] = ( q[a,h].kl[left(a,k),h] + kl[src(a,k),h].kr[c,h] + q[a,h].kr[c,h] ) / sqrt(F)
//   left(a,0) = src(a,0) = 0,  left(a,1) = max(a-1, 0),  src(a,1) = a-1 taken cyclically                       (:187-193)
//   links[a,k,c] = logsumexp_h( log_softmax_h(gate[a,:])[h] + log_softmax_{(k,c)}( z[a,:,:,h] )[k,c] )          (:168, 197-198)
// with masked entries -inf (:171-184) and rows without an allowed left option or right child -inf (:176-181, 199).
//
// Tiles: 32 parents x 32 right children per matrix instruction, the right children as the rows and the parents as the
// columns of the result, so that a lane holds 16 right children of ONE parent: the reductions over (k, c) of a parent
// are sums inside a lane, one exchange between the two halves of the wave and one through LDS between the waves.
// Operands are read as 16-byte chunks; which elements of the head dimension a lane feeds into which step of the
// instruction sequence is the same permutation for both operands, which a contraction does not see.
// fp16 chunks: v_mfma_f32_32x32x16_f16 (products of fp16 values are exact in fp32, accumulation in fp32: what the
// reference's `.to(float)` + einsum computes up to the order of the sum).  fp32 chunks: v_mfma_f32_32x32x2_f32.
#include "links_fused.hip.h"

namespace pcfgnat {
namespace {

// LDS of the forward kernel, in bytes: the query and left-key rows of the parent tile for all heads (row pitch: the row
// plus one chunk, which spreads the 32 rows of a column of chunks over the banks), the left-key row of node 0, and the
// per-parent tables.
inline size_t fused_fwd_lds_bytes(int L, int H, int F, int elem) {
    const size_t pitch = (size_t)H * F * elem + 16;
    const size_t nw = (size_t)(L + 31) / 32;
    return (2 * PT + 1) * pitch + sizeof(float) * ((size_t)PT * 2 * H + 2 * PT * H + (size_t)4 * PT * H * 2) +
           sizeof(unsigned) * (PT + 2 * nw + PT * nw);
}

// Forward.  grid (tiles of 32 parents, B); wave w of the workgroup takes the tiles w, w + 4, ... of 32 right children.
// links [B,L,2,L] and head_lse [B,L,H] (log-sum-exp over (k,c) of z per head) are written for every row.
// NCH: 16-byte chunks per lane of one head's row (F = 2 * NCH * elements per chunk).  The loops over the heads are
// kept rolled: the body of one head is a few hundred instructions, eight or sixteen copies of it would not stay in
// the instruction cache.  Inside the kernel all logarithms are to base 2 (log2(e) is folded into the scale).
template <typename T, int NCH>
__global__ __launch_bounds__(LF_NT) void links_fused_fwd_kernel(const T *__restrict__ q, const T *__restrict__ kl,
                                                               const T *__restrict__ kr, const float *__restrict__ gate,
                                                               const int64_t *__restrict__ prev_tokens, int64_t pad,
                                                               const unsigned char *__restrict__ ltm,
                                                               const unsigned char *__restrict__ rtm,
                                                               const unsigned char *__restrict__ main_chain,
                                                               float *__restrict__ links, float *__restrict__ lse_out,
                                                               unsigned *__restrict__ masks_out, int L, int H, float scale2) {
    constexpr int EPC = Chunk<T>::EPC, F = 2 * NCH * EPC;
    extern __shared__ uint4 lf_lds[];
    const int HF = H * F, cpr = HF / EPC, pitch = cpr + 1;  // chunks per row of all heads, row pitch in chunks
    const int nw = (L + 31) / 32;                           // tiles of 32 right children
    uint4 *sQ = lf_lds, *sK1 = sQ + PT * pitch, *sK0 = sK1 + PT * pitch;
    float *s_sab = reinterpret_cast<float *>(sK0 + pitch);  // [32][2H]: q.kl of both left options, scaled
    float *s_lg = s_sab + PT * 2 * H;                       // [32][H]: log-softmax of the gates
    float *s_lse = s_lg + PT * H;                           // [32][H]: log-sum-exp of z over (k,c)
    float *s_stat = s_lse + PT * H;                         // [4][32][H][2]: maximum and sum of every wave
    unsigned *s_flags = reinterpret_cast<unsigned *>(s_stat + 4 * PT * H * 2);  // [32]: 1 unusable, 2 / 4 left option 0 / 1 allowed
    unsigned *s_notpad = s_flags + PT, *s_cok = s_notpad + nw;                  // [nw] bits: not pad; not pad and on the main chain
    unsigned *s_allow = s_cok + nw;                                             // [32][nw] bits: right child allowed
    const int b = blockIdx.y, a0 = blockIdx.x * PT;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t *prev = prev_tokens + (size_t)b * L;

    // ---- everything the preamble reads from memory is requested first, in the order of its use
    // one byte of either tree mask per lane for the wave's parents 8w .. 8w+7 and a step of 64 children
    auto mask_bytes = [&](int base, unsigned char (&lv)[8], unsigned char (&rv)[8]) {
        const int c = base + lane;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int a = a0 + wave * 8 + i;
            const bool in = a < L && c < L;
            lv[i] = in ? ltm[(size_t)a * L + c] : (unsigned char)1;
            rv[i] = in ? rtm[(size_t)a * L + c] : (unsigned char)1;
        }
    };
    auto child_flags = [&](int base, bool &np, bool &ck) {
        const int c = base + tid;
        np = c < L && prev[c] != pad;
        ck = np && main_chain[c] != 0;
    };
    bool np_first, ck_first;
    child_flags(0, np_first, ck_first);
    unsigned char lv_first[8], rv_first[8];
    mask_bytes(0, lv_first, rv_first);
    float gate_first = 0.f;  // the gate logits of the tile's rows are contiguous
    {
        const int rows_in = min(PT, L - a0);
        if (tid < rows_in * H) gate_first = gate[((size_t)b * L + a0) * H + tid];
    }
    // the parent tile's query rows, the left-key rows src(a,1) and the left-key row of node 0, all heads: requested
    // here eight chunks of each per thread at a time, stored to LDS once the masks are done
    auto stage_load = [&](int i0, uint4 (&vq)[8], uint4 (&vk)[8]) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = i0 + u * LF_NT, pp = i / cpr, j = i - pp * cpr, a = a0 + pp;
            const int src = (a - 1 < 0) ? L - 1 : a - 1;
            vq[u] = vk[u] = make_uint4(0, 0, 0, 0);
            if (i < PT * cpr && a < L) {
                vq[u] = reinterpret_cast<const uint4 *>(q + ((size_t)b * L + a) * HF)[j];
                vk[u] = reinterpret_cast<const uint4 *>(kl + ((size_t)b * L + src) * HF)[j];
            }
        }
    };
    auto stage_store = [&](int i0, const uint4 (&vq)[8], const uint4 (&vk)[8]) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = i0 + u * LF_NT, pp = i / cpr, j = i - pp * cpr;
            if (i < PT * cpr) {
                sQ[pp * pitch + j] = vq[u];
                sK1[pp * pitch + j] = vk[u];
            }
        }
    };
    uint4 vq_first[8], vk_first[8];
    stage_load(tid, vq_first, vk_first);
    uint4 vk0_first = make_uint4(0, 0, 0, 0);
    if (tid < cpr) vk0_first = reinterpret_cast<const uint4 *>(kl + (size_t)b * L * HF)[tid];
    for (int i = tid; i < PT * H; i += LF_NT) {  // raw gate logits, parked where the waves' statistics go later
        const int rows_in = min(PT, L - a0);
        s_stat[i] = (i == tid) ? gate_first : (i < rows_in * H ? gate[((size_t)b * L + a0) * H + i] : 0.f);
    }
    // ---- per child: not pad, usable as a right child at all
    for (int base = 0; base < nw * 32; base += LF_NT) {
        bool np = np_first, ck = ck_first;
        if (base > 0) child_flags(base, np, ck);
        const unsigned long long bn = __ballot(np), bc = __ballot(ck);
        const int w0 = (base >> 5) + 2 * wave;
        if (lane == 0) {
            if (w0 < nw) {
                s_notpad[w0] = (unsigned)bn;
                s_cok[w0] = (unsigned)bc;
            }
            if (w0 + 1 < nw) {
                s_notpad[w0 + 1] = (unsigned)(bn >> 32);
                s_cok[w0 + 1] = (unsigned)(bc >> 32);
            }
        }
    }
    __syncthreads();
    // ---- per parent: the allowed right children as bits, whether any left / right entry is allowed (:171-181) and
    // whether its two left options are; the bits are collected by ballots, which are uniform over the wave, and lane i
    // keeps the words of parent 8w + i
    {
        unsigned mine_l = 0, mine_r = 0, mine_ok = 0;
        for (int base = 0; base < nw * 32; base += 64) {
            unsigned char lv[8], rv[8];
            if (base == 0) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    lv[i] = lv_first[i];
                    rv[i] = rv_first[i];
                }
            } else {
                mask_bytes(base, lv, rv);
            }
            const int w0 = base >> 5;
            const unsigned np0 = s_notpad[w0], ck0 = s_cok[w0];
            const unsigned np1 = (w0 + 1 < nw) ? s_notpad[w0 + 1] : 0u, ck1 = (w0 + 1 < nw) ? s_cok[w0 + 1] : 0u;
            unsigned ar0 = 0, ar1 = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const unsigned long long bl = __ballot(lv[i] == 0), br = __ballot(rv[i] == 0);
                const unsigned long long al = bl & (((unsigned long long)np1 << 32) | np0);
                const unsigned long long ar = br & (((unsigned long long)ck1 << 32) | ck0);
                const int a = a0 + wave * 8 + i, l1 = (a - 1 < 0) ? 0 : a - 1;
                unsigned ok = 0;
                if (base == 0) ok |= (unsigned)(al & 1ull) << 1;                                  // left option 0: node 0
                if (l1 >= base && l1 < base + 64) ok |= (unsigned)((al >> (l1 - base)) & 1ull) << 2;  // left option 1: node a-1
                if (lane == i) {
                    mine_l |= (al != 0) ? 1u : 0u;
                    mine_r |= (ar != 0) ? 1u : 0u;
                    mine_ok |= ok;
                    ar0 = (unsigned)ar;
                    ar1 = (unsigned)(ar >> 32);
                }
            }
            if (lane < 8) {
                s_allow[(wave * 8 + lane) * nw + w0] = ar0;
                if (w0 + 1 < nw) s_allow[(wave * 8 + lane) * nw + w0 + 1] = ar1;
            }
        }
        if (lane < 8) {
            const int pp = wave * 8 + lane, a = a0 + pp;
            s_flags[pp] = (a >= L || !mine_l || !mine_r) ? 1u : mine_ok;
        }
    }
    stage_store(tid, vq_first, vk_first);
    for (int i0 = tid + 8 * LF_NT; i0 < PT * cpr; i0 += 8 * LF_NT) {
        uint4 vq[8], vk[8];
        stage_load(i0, vq, vk);
        stage_store(i0, vq, vk);
    }
    if (tid < cpr) sK0[tid] = vk0_first;
    for (int j = tid + LF_NT; j < cpr; j += LF_NT) sK0[j] = reinterpret_cast<const uint4 *>(kl + (size_t)b * L * HF)[j];
    __syncthreads();
    if (masks_out != nullptr) {  // [B,L,1+nw]: the flags of every parent, then its allowed right children (for the backward)
        for (int i = tid; i < PT * (1 + nw); i += LF_NT) {
            const int pp = i / (1 + nw), w = i - pp * (1 + nw);
            if (a0 + pp < L) masks_out[((size_t)b * L + a0 + pp) * (1 + nw) + w] = (w == 0) ? s_flags[pp] : s_allow[pp * nw + w - 1];
        }
    }
    // ---- per (parent, head): the two q.kl terms and the log-softmax of the gates, in base 2
    {
        const int pp = tid & 31, a = a0 + pp;
        for (int h = tid >> 5; h < H; h += LF_NT / 32) {
            const uint4 *qrow = sQ + pp * pitch + h * (2 * NCH);
            const uint4 *k0row = sK0 + h * (2 * NCH), *k1row = (a == 0) ? k0row : sK1 + pp * pitch + h * (2 * NCH);  // left(0,1) = 0
            float d0 = 0.f, d1 = 0.f;
#pragma unroll
            for (int j = 0; j < 2 * NCH; j++) {
                const uint4 qv = qrow[j];
                d0 = Chunk<T>::dot(qv, k0row[j], d0);
                d1 = Chunk<T>::dot(qv, k1row[j], d1);
            }
            s_sab[pp * 2 * H + h] = d0 * scale2;
            s_sab[pp * 2 * H + H + h] = d1 * scale2;
        }
    }
    for (int i = tid; i < PT * H; i += LF_NT) {
        const int pp = i / H;
        const float *grow = s_stat + pp * H;
        float mx = NEG_INF_F;
        for (int j = 0; j < H; j++) mx = fmaxf(mx, grow[j]);
        float sum = 0.f;
        for (int j = 0; j < H; j++) sum += ex2((grow[j] - mx) * LF_LOG2E);
        s_lg[i] = (grow[i - pp * H] - mx) * LF_LOG2E - lg2(sum);
    }
    __syncthreads();

    const int p = lane & 31, kb = lane >> 5;
    const unsigned flags = s_flags[p];
    const bool ok0 = (flags & 2u) != 0, ok1 = (flags & 4u) != 0;
    // the right-key chunks of head h for the lane's row of tile ct (rows beyond the graph are masked by their allow bits)
    auto right_keys = [&](int ct, int h, uint4 (&ach)[NCH]) {
        const int crow = min(32 * ct + p, L - 1);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kr + ((size_t)b * L + crow) * HF + (size_t)h * F);
#pragma unroll
        for (int j = 0; j < NCH; j++) ach[j] = krow[2 * j + kb];
    };
    // 0 where the lane's right child r of tile ct may follow left option k, -inf where it may not
    float pen0[16], pen1[16];
    int pen_tile = -1;
    auto penalties = [&](int ct) {
        if (ct == pen_tile) return;
        pen_tile = ct;
        const unsigned allow = s_allow[p * nw + ct];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const bool c_ok = (allow >> acc_row(r, kb)) & 1u;
            pen0[r] = (ok0 && c_ok) ? 0.f : NEG_INF_F;
            pen1[r] = (ok1 && c_ok) ? 0.f : NEG_INF_F;
        }
    };
    // the scaled scores z[.][k] (base 2) of the lane's 16 right children for head h
    auto scores = [&](const uint4 (&ach)[NCH], int h, float (&z0)[16], float (&z1)[16]) {
        floatx16 ac, b1, b0;
#pragma unroll
        for (int r = 0; r < 16; r++) ac[r] = b1[r] = b0[r] = 0.f;
        const int hc = h * (2 * NCH);
        uint4 oq[NCH], o1[NCH], o0[NCH];  // all reads of the head in flight before the first product needs one
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            oq[j] = sQ[p * pitch + hc + 2 * j + kb];
            o1[j] = sK1[p * pitch + hc + 2 * j + kb];
            o0[j] = sK0[hc + 2 * j + kb];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            Chunk<T>::mma(ach[j], oq[j], ac);
            Chunk<T>::mma(ach[j], o1[j], b1);
            Chunk<T>::mma(ach[j], o0[j], b0);
        }
        const float sab0 = s_sab[p * 2 * H + h], sab1 = s_sab[p * 2 * H + H + h];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            z0[r] = __builtin_fmaf(b0[r] + ac[r], scale2, sab0) + pen0[r];
            z1[r] = __builtin_fmaf(b1[r] + ac[r], scale2, sab1) + pen1[r];
        }
    };
    const int ntw = (nw - wave + 3) / 4;  // tiles of this wave: wave, wave + 4, ...

    // ---- pass 1: per head the maximum and the sum of exponentials over (k, c); heads outside, the wave's tiles inside,
    // the chunks of the next step requested before the work of the current one
    {
        uint4 cur[NCH], nxt[NCH];
        if (ntw > 0) right_keys(wave, 0, cur);
        float m = LF_FLOOR, sacc = 0.f;
        const int steps = H * ntw;
        int h = 0, i = 0;  // step it = h * ntw + i
#pragma unroll 1
        for (int it = 0; it < steps; it++) {
            const int ct = wave + 4 * i;
            int hn = h, in = i + 1;  // the step after this one (the last step requests its own chunks again)
            if (in == ntw) {
                in = 0;
                hn = h + 1;
            }
            if (it + 1 == steps) {
                in = i;
                hn = h;
            }
            right_keys(wave + 4 * in, hn, nxt);
            penalties(ct);
            float z0[16], z1[16];
            scores(cur, h, z0, z1);
#pragma unroll
            for (int j = 0; j < NCH; j++) cur[j] = nxt[j];
            float mx = m;
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, fmaxf(z0[r], z1[r]));
            float sum = sacc * ex2(m - mx);
#pragma unroll
            for (int r = 0; r < 16; r++) sum += ex2(z0[r] - mx) + ex2(z1[r] - mx);
            sacc = sum;
            m = mx;
            if (i == ntw - 1) {  // the head is complete for this wave: the two halves of the wave hold the two halves of every tile's rows
                const float mo = __shfl_xor(m, 32), so = __shfl_xor(sacc, 32);
                const float mb = fmaxf(m, mo);
                if (kb == 0) {
                    s_stat[((wave * PT + p) * H + h) * 2 + 0] = mb;
                    s_stat[((wave * PT + p) * H + h) * 2 + 1] = sacc * ex2(m - mb) + so * ex2(mo - mb);
                }
                m = LF_FLOOR;
                sacc = 0.f;
            }
            h = hn;
            i = in;
        }
        if (ntw == 0 && kb == 0) {
            for (int h = 0; h < H; h++) {
                s_stat[((wave * PT + p) * H + h) * 2 + 0] = LF_FLOOR;
                s_stat[((wave * PT + p) * H + h) * 2 + 1] = 0.f;
            }
        }
    }
    __syncthreads();
    for (int i = tid; i < PT * H; i += LF_NT) {
        const int pp = i / H, h = i - pp * H;
        float mx = LF_FLOOR;
#pragma unroll
        for (int w = 0; w < 4; w++) mx = fmaxf(mx, s_stat[((w * PT + pp) * H + h) * 2]);
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) sum += s_stat[((w * PT + pp) * H + h) * 2 + 1] * ex2(s_stat[((w * PT + pp) * H + h) * 2] - mx);
        const float lse = (sum == 0.f) ? NEG_INF_F : mx + lg2(sum);
        // what pass 2 adds to the scores of this head; a head without any allowed entry has only -inf scores
        s_lse[i] = (sum == 0.f) ? 0.f : s_lg[i] - lse;
        if (a0 + pp < L) lse_out[((size_t)b * L + a0 + pp) * H + h] = (s_flags[pp] & 1u) ? NEG_INF_F : lse * LF_LN2;
    }
    __syncthreads();

    // ---- pass 2: mix the heads per entry; tiles outside, heads inside.  What a head adds to an entry is a probability
    // (its gate's share times its softmax: 2^t with t <= 0), so the sum over the heads can neither overflow nor lose its
    // largest term, and it is formed as it stands: one exponential and one addition per term.  Only where an allowed
    // entry's sum comes out below 2^-100 may terms have been lost to underflow; the wave then takes the tile again with a
    // running integral shift per entry (moving the sum to a new shift is an exact change of exponent), which covers the
    // whole range of the logarithmic form at nine more instructions per term.
    if (ntw > 0) {
        const int a = a0 + p;
        const bool unusable = (flags & 1u) != 0;
        const bool vec4 = (L & 3) == 0;
        // the links of tile ct from the sums and shifts of its entries: links = (shift + log2 sum) ln 2
        auto store_tile = [&](int ct, const float (&mx0)[16], const float (&sm0)[16], const float (&mx1)[16], const float (&sm1)[16]) {
            if (a >= L) return;
            float *out0 = links + ((size_t)b * L + a) * 2 * L, *out1 = out0 + L;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                float v0[4], v1[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int r = 4 * g + u;
                    v0[u] = (unusable || sm0[r] == 0.f) ? NEG_INF_F : (mx0[r] + lg2(sm0[r])) * LF_LN2;
                    v1[u] = (unusable || sm1[r] == 0.f) ? NEG_INF_F : (mx1[r] + lg2(sm1[r])) * LF_LN2;
                }
                const int c = 32 * ct + 8 * g + 4 * kb;  // the four rows of the group are consecutive right children
                if (vec4 && c < L) {
                    *reinterpret_cast<float4 *>(out0 + c) = make_float4(v0[0], v0[1], v0[2], v0[3]);
                    *reinterpret_cast<float4 *>(out1 + c) = make_float4(v1[0], v1[1], v1[2], v1[3]);
                } else {
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        if (c + u < L) {
                            out0[c + u] = v0[u];
                            out1[c + u] = v1[u];
                        }
                    }
                }
            }
        };
        // tile ct over all heads with the running shift (the rare second go; its keys are not requested ahead)
        auto shifted_tile = [&](int ct) {
            float mx0[16], sm0[16], mx1[16], sm1[16];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                mx0[r] = mx1[r] = LF_FLOOR;
                sm0[r] = sm1[r] = 0.f;
            }
            penalties(ct);
#pragma unroll 1
            for (int h = 0; h < H; h++) {
                uint4 keys[NCH];
                right_keys(ct, h, keys);
                float z0[16], z1[16];
                scores(keys, h, z0, z1);
                const float off = s_lse[p * H + h];
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float t0 = z0[r] + off, t1 = z1[r] + off;
                    const float n0 = fmaxf(mx0[r], __builtin_ceilf(t0)), n1 = fmaxf(mx1[r], __builtin_ceilf(t1));
                    sm0[r] = __builtin_ldexpf(sm0[r], (int)fmaxf(mx0[r] - n0, -256.f)) + ex2(t0 - n0);  // 2^-256 of a sum of H terms is 0
                    sm1[r] = __builtin_ldexpf(sm1[r], (int)fmaxf(mx1[r] - n1, -256.f)) + ex2(t1 - n1);
                    mx0[r] = n0;
                    mx1[r] = n1;
                }
            }
            store_tile(ct, mx0, sm0, mx1, sm1);
        };
        uint4 cur[NCH], nxt[NCH];
        right_keys(wave, 0, cur);
        float sm0[16], sm1[16];
#pragma unroll
        for (int r = 0; r < 16; r++) sm0[r] = sm1[r] = 0.f;
        const int steps = H * ntw;
        int h = 0, i = 0;  // step it = i * H + h
#pragma unroll 1
        for (int it = 0; it < steps; it++) {
            const int ct = wave + 4 * i;
            int hn = h + 1, in = i;
            if (hn == H) {
                hn = 0;
                in = i + 1;
            }
            if (it + 1 == steps) {
                in = i;
                hn = h;
            }
            right_keys(wave + 4 * in, hn, nxt);
            penalties(ct);
            float z0[16], z1[16];
            scores(cur, h, z0, z1);
#pragma unroll
            for (int j = 0; j < NCH; j++) cur[j] = nxt[j];
            const float off = s_lse[p * H + h];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                sm0[r] += ex2(z0[r] + off);
                sm1[r] += ex2(z1[r] + off);
            }
            if (h == H - 1) {  // the tile is complete
                bool thin = false;  // an allowed entry (penalty 0) with a sum so small that terms may have underflowed
#pragma unroll
                for (int r = 0; r < 16; r++)
                    thin = thin || (pen0[r] == 0.f && sm0[r] < LF_THIN_SUM) || (pen1[r] == 0.f && sm1[r] < LF_THIN_SUM);
                if (__ballot(thin && !unusable) != 0ull) {
                    shifted_tile(ct);
                } else {
                    float zero[16];
#pragma unroll
                    for (int r = 0; r < 16; r++) zero[r] = 0.f;
                    store_tile(ct, zero, sm0, zero, sm1);
                }
#pragma unroll
                for (int r = 0; r < 16; r++) sm0[r] = sm1[r] = 0.f;
            }
            h = hn;
            i = in;
        }
    }
}

int check_fused_args(const char *who, int dtype, int64_t B, int64_t L, int64_t H, int64_t F) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 2 && F >= 1, "%s: bad dimensions (B=%lld L=%lld F=%lld)", who, (long long)B, (long long)L, (long long)F);
    if (!(H == 1 || H == 2 || H == 4 || H == 8 || H == 16))
        return fail(PCFGNAT_EUNSUPPORTED, "%s: %lld attention heads (1, 2, 4, 8 and 16 are built)", who, (long long)H);
    if (dtype != PCFGNAT_F16 && dtype != PCFGNAT_F32)
        return fail(PCFGNAT_EUNSUPPORTED, "%s: chunks must be float16 or float32 (dtype code %d)", who, dtype);
    if (!fused_head_dim_built(dtype, F))
        return fail(PCFGNAT_EUNSUPPORTED, "%s: head dimension %lld (16, 32, 64, 128 are built for float16, 8, 16, 32, 64 for float32)", who,
                    (long long)F);
    PCFGNAT_REQUIRE(L <= 8192, "%s: graph too large (L <= 8192)", who);
    return PCFGNAT_OK;
}

template <typename T>
int launch_fused_fwd(const void *q, const void *kl, const void *kr, const float *gate, const int64_t *prev, int64_t pad,
                     const unsigned char *ltm, const unsigned char *rtm, const unsigned char *mc, float *links, float *lse,
                     unsigned *masks_out, int64_t B, int64_t L, int64_t H, int64_t F, hipStream_t s) {
    const size_t lds = fused_fwd_lds_bytes((int)L, (int)H, (int)F, (int)sizeof(T));
    if (lds > (size_t)160 * 1024)
        return fail(PCFGNAT_EUNSUPPORTED, "extract_links_fused_forward: %zu bytes of LDS needed (H*F = %lld, L = %lld)", lds,
                    (long long)(H * F), (long long)L);
    const dim3 grid((unsigned)((L + PT - 1) / PT), (unsigned)B);
    const float scale = LF_LOG2E / sqrtf((float)F);  // the kernel works in base 2
#define PCFGNAT_FUSED_FWD(nch)                                                                                                        \
    case nch: {                                                                                                                       \
        auto k = links_fused_fwd_kernel<T, nch>;                                                                                      \
        PCFGNAT_DYNAMIC_LDS(k, lds);                                                                                                  \
        hipLaunchKernelGGL(k, grid, dim3(LF_NT), lds, s, (const T *)q, (const T *)kl, (const T *)kr, gate, prev, pad, ltm, rtm, mc, links, \
                           lse, masks_out, (int)L, (int)H, scale);                                                                               \
        break;                                                                                                                        \
    }
    switch (F / (2 * Chunk<T>::EPC)) {
        PCFGNAT_FUSED_FWD(1)
        PCFGNAT_FUSED_FWD(2)
        PCFGNAT_FUSED_FWD(4)
        PCFGNAT_FUSED_FWD(8)
    }
#undef PCFGNAT_FUSED_FWD
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

extern "C" int pcfgnat_extract_links_fused_supported(int dtype, int64_t L, int64_t H, int64_t F) {
    if (!(H == 1 || H == 2 || H == 4 || H == 8 || H == 16) || L < 2 || L > 8192) return 0;
    if (dtype != PCFGNAT_F16 && dtype != PCFGNAT_F32) return 0;
    const int elem = dtype == PCFGNAT_F16 ? 2 : 4;
    if (!fused_head_dim_built(dtype, F)) return 0;
    return fused_fwd_lds_bytes((int)L, (int)H, (int)F, elem) <= (size_t)160 * 1024 ? 1 : 0;
}

extern "C" int pcfgnat_extract_links_fused_forward(const void *query_chunks, const void *key_chunks_left, const void *key_chunks_right,
                                                   int dtype, const float *gate_logits, const int64_t *prev_output_tokens,
                                                   int64_t pad_index, const unsigned char *left_tree_mask,
                                                   const unsigned char *right_tree_mask, const unsigned char *main_chain, float *links,
                                                   float *head_lse, unsigned *tile_masks, int64_t B, int64_t L, int64_t H, int64_t F,
                                                   void *stream) {
    int rc = check_fused_args("extract_links_fused_forward", dtype, B, L, H, F);
    if (rc != PCFGNAT_OK) return rc;
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(query_chunks && key_chunks_left && key_chunks_right && gate_logits && prev_output_tokens && left_tree_mask &&
                        right_tree_mask && main_chain && links && head_lse,
                    "extract_links_fused_forward: null pointer");
    PCFGNAT_REQUIRE((((uintptr_t)query_chunks | (uintptr_t)key_chunks_left | (uintptr_t)key_chunks_right | (uintptr_t)links) & 15) == 0,
                    "extract_links_fused_forward: chunks and links must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PCFGNAT_F16)
        return launch_fused_fwd<__half>(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad_index,
                                        left_tree_mask, right_tree_mask, main_chain, links, head_lse, tile_masks, B, L, H, F, s);
    return launch_fused_fwd<float>(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad_index,
                                   left_tree_mask, right_tree_mask, main_chain, links, head_lse, tile_masks, B, L, H, F, s);
}
