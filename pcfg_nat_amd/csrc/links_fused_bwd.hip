// Backward of the link scorer of PCFG-NAT (reference fs_plugins/models/glat_decomposed_with_link_two_hands_tri_pcfg.py:
// 140-201, `extract_links`, what autograd derives from it) with every product on the matrix cores inside the kernels:
// the scores z are recomputed from the chunks tile by tile, their gradient dz exists only in registers and LDS.
//
// With w[a,k,c,h] = exp(log gate_h + log softmax_h(z)[k,c] - links[a,k,c]) (the share of head h in a link) and G the
// upstream gradient:
//   dg[a,h]       = sum_{k,c} G w                      d gate_logits[a,h] = dg[a,h] - gate_h * sum_h' dg[a,h']
//   dz[a,k,c,h]   = (G w - softmax_h(z)[k,c] dg[a,h]) / sqrt(F)
//   d q[a,h]      = sum_c (dz[a,0,c] + dz[a,1,c]) kr[c,h] + ds[a,0] kl[0,h] + ds[a,1] kl[left(a,1),h],  ds[a,k] = sum_c dz[a,k,c]
//   d kl[j,h]     = sum_c dz[a,1,c] kr[c,h] + ds[a,1] q[a,h]  for the parent a with src(a,1) = j (a = j+1 cyclically; the
//                   q term goes to left(a,1), which differs for a = 0), plus for j = 0 the null option of every parent:
//                   sum_a ( sum_c dz[a,0,c] kr[c,h] + ds[a,0] q[a,h] )
//   d kr[c,h]     = sum_a ( (dz[a,0,c] + dz[a,1,c]) q[a,h] + dz[a,0,c] kl[0,h] + dz[a,1,c] kl[src(a,1),h] )
// Three launches; the masks of every parent come from the forward.  The four waves of a workgroup work on four heads of
// the same tiles and share nothing but the reading of links and G:
//   parents:  one wave per (sentence, head, tile of 32 parents) runs over the tiles of right children twice (dg, then
//             dz) and leaves d q, d kl (all rows but row 0), d gate and, for the other two launches, dg and ds;
//   children: one wave per (sentence, head, tile of 32 right children) runs over the tiles of parents and leaves d kr
//             and the column sums of dz[.,0,.];
//   row 0:    d kl[0,h] from what the other two left.
// The products with dz run in fp32 (v_mfma_f32_32x32x2_f32, dz as one operand straight from the accumulator layout or
// transposed through LDS); the scores use the same chunks and instructions as the forward.
#include "links_fused.hip.h"

namespace pcfgnat {
namespace {

// ---- workspace of one backward call (floats), in this order
struct BwdWorkspace {
    float *dg;    // [B,L,H]
    float *ds;    // [B,H,L,2]
    float *cs;    // [B,H,L]   column sums of dz[.,0,.]
    float *row0;  // [B,H,F]   d kl[0,h] as far as the parents' launch gets
    float *lg;    // [B,L,H]   log2 of the gates
};
inline size_t bwd_workspace_words(int64_t B, int64_t L, int64_t H, int64_t F) {
    return (size_t)(2 * B * L * H + B * H * L * 2 + B * H * L + B * H * F);
}
inline BwdWorkspace bwd_workspace(float *ws, int64_t B, int64_t L, int64_t H, int64_t F) {
    BwdWorkspace w;
    w.dg = ws;
    w.ds = w.dg + B * L * H;
    w.cs = w.ds + B * H * L * 2;
    w.row0 = w.cs + B * H * L;
    w.lg = w.row0 + B * H * F;
    return w;
}

// What a wave needs of one (parent, head) besides the chunks: in base 2.
struct ParentTerms {
    float sab0, sab1;  // q.kl of the two left options, scaled
    float off;         // log gate - lse (0 where the head has no allowed entry: its scores are all -inf)
    float lse2;        // lse (0 likewise)
    float lg2v;        // log gate
};
__device__ __forceinline__ void gate_terms(const float *__restrict__ grow, int H, int h, float lse, ParentTerms &pt) {
    float mx = NEG_INF_F;
    for (int j = 0; j < H; j++) mx = fmaxf(mx, grow[j]);
    float sum = 0.f;
    for (int j = 0; j < H; j++) sum += ex2((grow[j] - mx) * LF_LOG2E);
    pt.lg2v = (grow[h] - mx) * LF_LOG2E - lg2(sum);
    pt.lse2 = (lse == NEG_INF_F) ? 0.f : lse * LF_LOG2E;
    pt.off = (lse == NEG_INF_F) ? 0.f : pt.lg2v - pt.lse2;
}

// d z of the lane's 16 right children for both left options from the scores, the upstream gradient and the links
// (natural logarithms) of the same entries; gsum collects G over the finite links.  FIRST: only dg is wanted.
template <bool FIRST>
__device__ __forceinline__ void entry_gradients(const float (&z0)[16], const float (&z1)[16], const float (&g0)[16], const float (&g1)[16],
                                                const float (&l0)[16], const float (&l1)[16], const ParentTerms &pt, float dgv,
                                                float scale, float &dg, float &gsum, float (&dz0)[16], float (&dz1)[16]) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const bool f0 = l0[r] != NEG_INF_F, f1 = l1[r] != NEG_INF_F;  // masked entries are constants: no gradient
        const float w0 = ex2((z0[r] + pt.off) - (f0 ? l0[r] * LF_LOG2E : 0.f));
        const float w1 = ex2((z1[r] + pt.off) - (f1 ? l1[r] * LF_LOG2E : 0.f));
        const float gw0 = f0 ? g0[r] * w0 : 0.f, gw1 = f1 ? g1[r] * w1 : 0.f;
        if (FIRST) {
            dg += gw0 + gw1;
            gsum += (f0 ? g0[r] : 0.f) + (f1 ? g1[r] : 0.f);
        } else {
            dz0[r] = (gw0 - ex2(z0[r] - pt.lse2) * dgv) * scale;
            dz1[r] = (gw1 - ex2(z1[r] - pt.lse2) * dgv) * scale;
        }
    }
}

// ---- the links and the upstream gradient of a tile of 32 parents x 32 right children, both left options: read once by
// the four waves of a workgroup (which work on four heads of the same tile) and handed on through LDS, the next tile in
// flight while the current one is worked on.  Layout [array][parent][k * 32 + right child], row pitch 68 floats.
constexpr int ENT_PITCH = 68, ENT_FLOATS = 2 * PT * ENT_PITCH;  // one buffer: links, then the gradient
struct EntryLoad {
    float4 v[4];
};
// thread tid requests its four float4 of the tile (parents a0.., right children c0..); entries beyond the graph read as
// -inf (links) and 0 (gradient)
__device__ __forceinline__ void entries_request(const float *__restrict__ links, const float *__restrict__ G, int b, int a0, int c0, int L,
                                                bool vec4, int tid, EntryLoad &e) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int idx = tid + LF_NT * u, arr = idx >> 9, rem = idx & 511, pp = rem >> 4, k = (rem >> 3) & 1, c = c0 + 4 * (rem & 7);
        const float fill = arr == 0 ? NEG_INF_F : 0.f;
        const int a = a0 + pp;
        const float *row = (arr == 0 ? links : G) + (((size_t)b * L + (a < L ? a : 0)) * 2 + k) * L;
        if (a < L && vec4 && c < L) {
            e.v[u] = *reinterpret_cast<const float4 *>(row + c);
        } else {
            e.v[u].x = (a < L && c + 0 < L) ? row[c + 0] : fill;
            e.v[u].y = (a < L && c + 1 < L) ? row[c + 1] : fill;
            e.v[u].z = (a < L && c + 2 < L) ? row[c + 2] : fill;
            e.v[u].w = (a < L && c + 3 < L) ? row[c + 3] : fill;
        }
    }
}
__device__ __forceinline__ void entries_store(float *buf, int tid, const EntryLoad &e) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int idx = tid + LF_NT * u, arr = idx >> 9, rem = idx & 511, pp = rem >> 4, k = (rem >> 3) & 1, c4 = rem & 7;
        *reinterpret_cast<float4 *>(buf + (arr * PT + pp) * ENT_PITCH + k * 32 + 4 * c4) = e.v[u];
    }
}
// the 16 entries of lane (p, kb) for left option k: rows acc_row(r, kb) of the tile, four groups of four consecutive children
__device__ __forceinline__ void entries_read(const float *buf, int arr, int p, int k, int kb, float (&v)[16]) {
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float4 x = *reinterpret_cast<const float4 *>(buf + (arr * PT + p) * ENT_PITCH + k * 32 + 8 * g + 4 * kb);
        v[4 * g + 0] = x.x;
        v[4 * g + 1] = x.y;
        v[4 * g + 2] = x.z;
        v[4 * g + 3] = x.w;
    }
}

// LDS per wave, in chunks: TILES tiles of 32 rows of one head (row pitch: the row plus one chunk) and one more row.
template <int NCH, int TILES>
constexpr int bwd_wave_chunks() {
    return TILES * PT * (2 * NCH + 1) + (2 * NCH + 1);
}
constexpr int BWD_TD_PITCH = 33;  // floats per row of a transposed 32 x 32 tile

// ---- parents' launch.  grid (tiles of 32 parents, groups of four heads, B); wave w of the workgroup takes head
// 4 * group + w (a wave without a head still helps to move the entries).  masks: [B,L,1+nw] words as the forward left
// them (flags, then the allowed right children).
template <typename T, int NCH>
__global__ __launch_bounds__(LF_NT) void links_fused_bwd_parents_kernel(
    const T *__restrict__ q, const T *__restrict__ kl, const T *__restrict__ kr, const float *__restrict__ gate,
    const float *__restrict__ head_lse, const float *__restrict__ links, const float *__restrict__ G, const unsigned *__restrict__ masks,
    T *__restrict__ dq, T *__restrict__ dkl, float *__restrict__ dgate, BwdWorkspace ws, int L, int H, float scale2, float scale) {
    constexpr int EPC = Chunk<T>::EPC, F = 2 * NCH * EPC, FT = (F + 31) / 32, RPC = 2 * NCH + 1;
    extern __shared__ uint4 lb_lds[];
    const int nw = (L + 31) / 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.z, a0 = blockIdx.x * PT, h = blockIdx.y * 4 + wave;
    const bool active = h < H;
    uint4 *tQ = lb_lds + wave * bwd_wave_chunks<NCH, 3>(), *tK1 = tQ + PT * RPC, *tKr = tK1 + PT * RPC, *tK0 = tKr + PT * RPC;
    float *s_ent = reinterpret_cast<float *>(lb_lds + 4 * bwd_wave_chunks<NCH, 3>());  // two buffers of entries
    float *s_ds = s_ent + 2 * ENT_FLOATS + wave * 64;                                 // [2][32] per wave
    const int p = lane & 31, kb = lane >> 5, a = a0 + p;
    const bool in = a < L;
    const int ai = in ? a : 0, hh = active ? h : 0;
    const int HF = H * F;
    const bool vec4 = (L & 3) == 0;
    EntryLoad ent;
    entries_request(links, G, b, a0, 0, L, vec4, tid, ent);
    const unsigned *mrow = masks + ((size_t)b * L + ai) * (1 + nw);
    const unsigned flags = in ? mrow[0] : 1u;
    // ---- the wave's rows of head h: query, left key src(a,1), left key of node 0; chunks 2j + kb of row p per lane
    ParentTerms pt;
    {
        float sab0 = 0.f, sab1 = 0.f;
        const int src = (a - 1 < 0) ? L - 1 : a - 1;
        const uint4 *qrow = reinterpret_cast<const uint4 *>(q + ((size_t)b * L + ai) * HF + (size_t)hh * F);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kl + ((size_t)b * L + (in ? src : 0)) * HF + (size_t)hh * F);
        const uint4 *k0row = reinterpret_cast<const uint4 *>(kl + (size_t)b * L * HF + (size_t)hh * F);
        uint4 vq[NCH], vk[NCH], v0[NCH];
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            vq[j] = in ? qrow[2 * j + kb] : make_uint4(0, 0, 0, 0);
            vk[j] = in ? krow[2 * j + kb] : make_uint4(0, 0, 0, 0);
            v0[j] = k0row[2 * j + kb];
        }
        const float lse = head_lse[((size_t)b * L + ai) * H + hh];
        gate_terms(gate + ((size_t)b * L + ai) * H, H, hh, lse, pt);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            tQ[p * RPC + 2 * j + kb] = vq[j];
            tK1[p * RPC + 2 * j + kb] = vk[j];
            if (p == 0) tK0[2 * j + kb] = v0[j];
            sab0 = Chunk<T>::dot(vq[j], v0[j], sab0);
            sab1 = Chunk<T>::dot(vq[j], a == 0 ? v0[j] : vk[j], sab1);  // left(0,1) = 0, not the cyclic src
        }
        sab0 += __shfl_xor(sab0, 32);
        sab1 += __shfl_xor(sab1, 32);
        pt.sab0 = sab0 * scale2;
        pt.sab1 = sab1 * scale2;
    }
    const bool usable = (flags & 1u) == 0;
    const bool ok0 = usable && (flags & 2u) != 0, ok1 = usable && (flags & 4u) != 0;

    auto right_keys = [&](int ct, uint4 (&ach)[NCH], unsigned &allow) {
        const int crow = min(32 * ct + p, L - 1);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kr + ((size_t)b * L + crow) * HF + (size_t)hh * F);
#pragma unroll
        for (int j = 0; j < NCH; j++) ach[j] = krow[2 * j + kb];
        allow = in ? mrow[1 + ct] : 0u;
    };
    // scores (base 2) of the lane's 16 right children, -inf where masked
    auto scores = [&](const uint4 (&ach)[NCH], unsigned allow, float (&z0)[16], float (&z1)[16]) {
        uint4 oq[NCH], o1[NCH], o0[NCH];
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            oq[j] = tQ[p * RPC + 2 * j + kb];
            o1[j] = tK1[p * RPC + 2 * j + kb];
            o0[j] = tK0[2 * j + kb];
        }
        floatx16 ac, b1, b0;
#pragma unroll
        for (int r = 0; r < 16; r++) ac[r] = b1[r] = b0[r] = 0.f;
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            Chunk<T>::mma(ach[j], oq[j], ac);
            Chunk<T>::mma(ach[j], o1[j], b1);
            Chunk<T>::mma(ach[j], o0[j], b0);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const bool c_ok = (allow >> acc_row(r, kb)) & 1u;
            z0[r] = (ok0 && c_ok) ? __builtin_fmaf(b0[r] + ac[r], scale2, pt.sab0) : NEG_INF_F;
            z1[r] = (ok1 && c_ok) ? __builtin_fmaf(b1[r] + ac[r], scale2, pt.sab1) : NEG_INF_F;
        }
    };

    floatx16 accQ[FT], accK[FT];
#pragma unroll
    for (int t = 0; t < FT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) accQ[t][r] = accK[t][r] = 0.f;
    float dg = 0.f, gsum = 0.f, ds0 = 0.f, ds1 = 0.f;
    uint4 cur[NCH], nxt[NCH];
    unsigned allow_cur, allow_nxt;
    right_keys(0, cur, allow_cur);
    entries_store(s_ent, tid, ent);
    __syncthreads();
    // ---- two runs over the tiles of right children as one sequence of steps: the first run gives dg = sum G w (and the sum
    // of G over the finite links), the second dz and its products with the right keys
#pragma unroll 1
    for (int s = 0; s < 2 * nw; s++) {
        const int sn = min(s + 1, 2 * nw - 1), ctn = sn < nw ? sn : sn - nw;  // the tile of step s is s mod nw
        entries_request(links, G, b, a0, 32 * ctn, L, vec4, tid, ent);
        right_keys(ctn, nxt, allow_nxt);
        const float *buf = s_ent + (s & 1) * ENT_FLOATS;
        if (active) {
            float g0[16], g1[16], l0[16], l1[16], z0[16], z1[16], dz0[16], dz1[16];
            entries_read(buf, 0, p, 0, kb, l0);
            entries_read(buf, 0, p, 1, kb, l1);
            entries_read(buf, 1, p, 0, kb, g0);
            entries_read(buf, 1, p, 1, kb, g1);
            scores(cur, allow_cur, z0, z1);
            if (s < nw) {
                entry_gradients<true>(z0, z1, g0, g1, l0, l1, pt, 0.f, scale, dg, gsum, dz0, dz1);
                if (s == nw - 1) {
                    dg += __shfl_xor(dg, 32);
                    gsum += __shfl_xor(gsum, 32);
                    if (in && kb == 0) {
                        // (the sum over the heads of dg is the sum of G over the finite links)
                        dgate[((size_t)b * L + a) * H + h] = dg - ex2(pt.lg2v) * gsum;
                        ws.dg[((size_t)b * L + a) * H + h] = dg;
                        ws.lg[((size_t)b * L + a) * H + h] = pt.lg2v;
                    }
                }
            } else {
                // the right keys of the tile as a table [row][element] for the products below
#pragma unroll
                for (int j = 0; j < NCH; j++) tKr[p * RPC + 2 * j + kb] = cur[j];
                float unused_dg = 0.f, unused_gs = 0.f;
                entry_gradients<false>(z0, z1, g0, g1, l0, l1, pt, dg, scale, unused_dg, unused_gs, dz0, dz1);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    ds0 += dz0[r];
                    ds1 += dz1[r];
                }
                // d q[p][f] += sum_c (dz0 + dz1)[p][c] kr[c][f],  d kl[src(p)][f] += sum_c dz1[p][c] kr[c][f]: dz is already
                // laid out as the row operand (lane: parent p, step r: right child acc_row(r, kb)); lane (f, kb) supplies
                // kr[acc_row(r, kb)][f]
                float kv[FT][16];
#pragma unroll
                for (int r = 0; r < 16; r++)
#pragma unroll
                    for (int t = 0; t < FT; t++) kv[t][r] = (32 * t + p < F) ? Chunk<T>::elem(tKr + acc_row(r, kb) * RPC, 32 * t + p) : 0.f;
#pragma unroll
                for (int r = 0; r < 16; r++) {
#pragma unroll
                    for (int t = 0; t < FT; t++) {
                        accQ[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(dz0[r] + dz1[r], kv[t][r], accQ[t], 0, 0, 0);
                        accK[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(dz1[r], kv[t][r], accK[t], 0, 0, 0);
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NCH; j++) cur[j] = nxt[j];
        allow_cur = allow_nxt;
        entries_store(s_ent + ((s + 1) & 1) * ENT_FLOATS, tid, ent);
        __syncthreads();
    }
    if (!active) return;
    ds0 += __shfl_xor(ds0, 32);
    ds1 += __shfl_xor(ds1, 32);
    if (kb == 0) {
        s_ds[p] = ds0;
        s_ds[32 + p] = ds1;
        if (in) {
            ws.ds[(((size_t)b * H + h) * L + a) * 2 + 0] = ds0;
            ws.ds[(((size_t)b * H + h) * L + a) * 2 + 1] = ds1;
        }
    }
    // ---- the q.kl terms and the stores: lane (f, kb) holds the parents acc_row(r, kb) of column f
#pragma unroll
    for (int t = 0; t < FT; t++) {
        const int f = 32 * t + p;
        if (f >= F) continue;
        const float k0f = Chunk<T>::elem(tK0, f);
        float d0[16], d1[16], k1f[16], qf[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {  // every read of the tile before the first use
            const int pr = acc_row(r, kb);
            d0[r] = s_ds[pr];
            d1[r] = s_ds[32 + pr];
            k1f[r] = Chunk<T>::elem(tK1 + pr * RPC, f);
            qf[r] = Chunk<T>::elem(tQ + pr * RPC, f);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int ar = a0 + acc_row(r, kb);
            if (ar >= L) continue;
            dq[((size_t)b * L + ar) * HF + (size_t)h * F + f] = Chunk<T>::cast(accQ[t][r] + d0[r] * k0f + d1[r] * (ar == 0 ? k0f : k1f[r]));
            const float dk = accK[t][r] + (ar >= 1 ? d1[r] * qf[r] : 0.f);
            const int src = (ar - 1 < 0) ? L - 1 : ar - 1;
            if (src == 0) ws.row0[((size_t)b * H + h) * F + f] = dk;  // completed by the last launch
            else dkl[((size_t)b * L + src) * HF + (size_t)h * F + f] = Chunk<T>::cast(dk);
        }
    }
}

// ---- children's launch.  grid (tiles of 32 right children, groups of four heads, B); wave w takes head 4 * group + w.
template <typename T, int NCH>
__global__ __launch_bounds__(LF_NT) void links_fused_bwd_children_kernel(
    const T *__restrict__ q, const T *__restrict__ kl, const T *__restrict__ kr, const float *__restrict__ head_lse,
    const float *__restrict__ links, const float *__restrict__ G, const unsigned *__restrict__ masks, T *__restrict__ dkr, BwdWorkspace ws,
    int L, int H, float scale2, float scale) {
    constexpr int EPC = Chunk<T>::EPC, F = 2 * NCH * EPC, FT = (F + 31) / 32, RPC = 2 * NCH + 1;
    extern __shared__ uint4 lb_lds[];
    const int nw = (L + 31) / 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.z, ct = blockIdx.x, c0 = ct * PT, h = blockIdx.y * 4 + wave;
    const bool active = h < H;
    const int hh = active ? h : 0;
    uint4 *tQ = lb_lds + wave * bwd_wave_chunks<NCH, 2>(), *tK1 = tQ + PT * RPC, *tK0 = tK1 + PT * RPC;
    float *s_ent = reinterpret_cast<float *>(lb_lds + 4 * bwd_wave_chunks<NCH, 2>());
    float *tD = s_ent + 2 * ENT_FLOATS + wave * (2 * PT * BWD_TD_PITCH + PT);  // [2][32][33], [32]
    float *s_cs = tD + 2 * PT * BWD_TD_PITCH;
    const int p = lane & 31, kb = lane >> 5;
    const int HF = H * F;
    const bool vec4 = (L & 3) == 0;
    EntryLoad ent;
    entries_request(links, G, b, 0, c0, L, vec4, tid, ent);
    // the right keys of the wave's tile (the row operand of the scores) stay in registers; the left key of node 0 in LDS
    uint4 akr[NCH];
    {
        const int crow = min(c0 + p, L - 1);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kr + ((size_t)b * L + crow) * HF + (size_t)hh * F);
        const uint4 *k0row = reinterpret_cast<const uint4 *>(kl + (size_t)b * L * HF + (size_t)hh * F);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            akr[j] = krow[2 * j + kb];
            if (p == 0) tK0[2 * j + kb] = k0row[2 * j + kb];
        }
    }
    // what the step for parent tile pt needs from memory besides the entries
    struct ParentLoad {
        uint4 vq[NCH], vk[NCH];
        unsigned flags, allow;
        float lse, dgv, lgv;
    };
    auto parent_request = [&](int pt, ParentLoad &pl) {
        const int a = 32 * pt + p;
        const bool in = a < L;
        const int ai = in ? a : 0, src = (ai - 1 < 0) ? L - 1 : ai - 1;
        const uint4 *qrow = reinterpret_cast<const uint4 *>(q + ((size_t)b * L + ai) * HF + (size_t)hh * F);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kl + ((size_t)b * L + src) * HF + (size_t)hh * F);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            pl.vq[j] = qrow[2 * j + kb];
            pl.vk[j] = krow[2 * j + kb];
        }
        const unsigned *mrow = masks + ((size_t)b * L + ai) * (1 + nw);
        pl.flags = in ? mrow[0] : 1u;  // parents beyond the graph count as unusable
        pl.allow = in ? mrow[1 + ct] : 0u;
        pl.lse = head_lse[((size_t)b * L + ai) * H + hh];
        pl.dgv = in ? ws.dg[((size_t)b * L + ai) * H + hh] : 0.f;
        pl.lgv = in ? ws.lg[((size_t)b * L + ai) * H + hh] : 0.f;
    };
    floatx16 accR[FT];
#pragma unroll
    for (int t = 0; t < FT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) accR[t][r] = 0.f;
    float cs0 = 0.f;
    ParentLoad cur, nxt;
    parent_request(0, cur);
    entries_store(s_ent, tid, ent);
    __syncthreads();
#pragma unroll 1
    for (int pt = 0; pt < nw; pt++) {
        const int ptn = min(pt + 1, nw - 1);
        entries_request(links, G, b, 32 * ptn, c0, L, vec4, tid, ent);
        parent_request(ptn, nxt);
        const float *buf = s_ent + (pt & 1) * ENT_FLOATS;
        if (active) {
            const int a = 32 * pt + p;
            ParentTerms ptm;
            ptm.lg2v = cur.lgv;
            ptm.lse2 = (cur.lse == NEG_INF_F) ? 0.f : cur.lse * LF_LOG2E;
            ptm.off = (cur.lse == NEG_INF_F) ? 0.f : ptm.lg2v - ptm.lse2;
            // the parents' rows as chunks (column operand of the scores) and as tables for the products
            float sab0 = 0.f, sab1 = 0.f;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                tQ[p * RPC + 2 * j + kb] = cur.vq[j];
                tK1[p * RPC + 2 * j + kb] = cur.vk[j];
                const uint4 v0 = tK0[2 * j + kb];
                sab0 = Chunk<T>::dot(cur.vq[j], v0, sab0);
                sab1 = Chunk<T>::dot(cur.vq[j], a == 0 ? v0 : cur.vk[j], sab1);
            }
            sab0 += __shfl_xor(sab0, 32);
            sab1 += __shfl_xor(sab1, 32);
            ptm.sab0 = sab0 * scale2;
            ptm.sab1 = sab1 * scale2;
            const bool usable = (cur.flags & 1u) == 0;
            const bool ok0 = usable && (cur.flags & 2u) != 0, ok1 = usable && (cur.flags & 4u) != 0;
            float z0[16], z1[16], dz0[16], dz1[16];
            {
                floatx16 ac, b1, b0;
#pragma unroll
                for (int r = 0; r < 16; r++) ac[r] = b1[r] = b0[r] = 0.f;
#pragma unroll
                for (int j = 0; j < NCH; j++) {
                    Chunk<T>::mma(akr[j], cur.vq[j], ac);
                    Chunk<T>::mma(akr[j], cur.vk[j], b1);
                    Chunk<T>::mma(akr[j], tK0[2 * j + kb], b0);
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const bool c_ok = (cur.allow >> acc_row(r, kb)) & 1u;
                    z0[r] = (ok0 && c_ok) ? __builtin_fmaf(b0[r] + ac[r], scale2, ptm.sab0) : NEG_INF_F;
                    z1[r] = (ok1 && c_ok) ? __builtin_fmaf(b1[r] + ac[r], scale2, ptm.sab1) : NEG_INF_F;
                }
            }
            float g0[16], g1[16], l0[16], l1[16];
            entries_read(buf, 0, p, 0, kb, l0);
            entries_read(buf, 0, p, 1, kb, l1);
            entries_read(buf, 1, p, 0, kb, g0);
            entries_read(buf, 1, p, 1, kb, g1);
            float unused_dg = 0.f, unused_gs = 0.f;
            entry_gradients<false>(z0, z1, g0, g1, l0, l1, ptm, cur.dgv, scale, unused_dg, unused_gs, dz0, dz1);
            // transposed through LDS: tD[k][parent][right child], read back with the right child as the row of the operand
#pragma unroll
            for (int r = 0; r < 16; r++) {
                tD[p * BWD_TD_PITCH + acc_row(r, kb)] = dz0[r];
                tD[(PT + p) * BWD_TD_PITCH + acc_row(r, kb)] = dz1[r];
            }
            // d kr[c][f] += sum_p (dz0 + dz1)[p][c] q[p][f] + sum_p dz1[p][c] kl[src(p)][f]: lane (c, kb) supplies the gradients
            // of parent 2 s + kb in step s, lane (f, kb) the elements of that parent's rows
            float d0v[16], d1v[16], qv[FT][16], kv[FT][16];
#pragma unroll
            for (int s = 0; s < 16; s++) {  // every read before the first product
                const int pp = 2 * s + kb;
                d0v[s] = tD[pp * BWD_TD_PITCH + p];
                d1v[s] = tD[(PT + pp) * BWD_TD_PITCH + p];
#pragma unroll
                for (int t = 0; t < FT; t++) {
                    const int f = 32 * t + p;
                    qv[t][s] = (f < F) ? Chunk<T>::elem(tQ + pp * RPC, f) : 0.f;
                    kv[t][s] = (f < F) ? Chunk<T>::elem(tK1 + pp * RPC, f) : 0.f;
                }
            }
#pragma unroll
            for (int s = 0; s < 16; s++) {
                cs0 += d0v[s];
#pragma unroll
                for (int t = 0; t < FT; t++) {
                    accR[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(d0v[s] + d1v[s], qv[t][s], accR[t], 0, 0, 0);
                    accR[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(d1v[s], kv[t][s], accR[t], 0, 0, 0);
                }
            }
        }
        cur = nxt;
        entries_store(s_ent + ((pt + 1) & 1) * ENT_FLOATS, tid, ent);
        __syncthreads();
    }
    if (!active) return;
    cs0 += __shfl_xor(cs0, 32);  // lane (c, kb) summed the parents of its half
    if (kb == 0) {
        s_cs[p] = cs0;
        if (c0 + p < L) ws.cs[((size_t)b * H + h) * L + c0 + p] = cs0;
    }
    // ---- the null option's left key and the stores: lane (f, kb) holds the right children acc_row(r, kb) of column f
#pragma unroll
    for (int t = 0; t < FT; t++) {
        const int f = 32 * t + p;
        if (f >= F) continue;
        const float k0f = Chunk<T>::elem(tK0, f);
        float csr[16];
#pragma unroll
        for (int r = 0; r < 16; r++) csr[r] = s_cs[acc_row(r, kb)];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int c = c0 + acc_row(r, kb);
            if (c < L) dkr[((size_t)b * L + c) * HF + (size_t)h * F + f] = Chunk<T>::cast(accR[t][r] + csr[r] * k0f);
        }
    }
}

// ---- d kl[0,h]: what the parents' launch left, the null option of every parent and parent 0's clamped left option.
// grid (B * H), 256 threads: element f by thread f % F, the sums over the rows split over the 256 / F groups of threads.
template <typename T>
__global__ __launch_bounds__(256) void links_fused_bwd_row0_kernel(const T *__restrict__ q, const T *__restrict__ kr, T *__restrict__ dkl,
                                                                  BwdWorkspace ws, int L, int H, int F) {
    __shared__ float s_part[256];
    const int bh = blockIdx.x, b = bh / H, h = bh - b * H;
    const int tid = threadIdx.x, f = tid % F, grp = tid / F, groups = 256 / F;
    const size_t HF = (size_t)H * F;
    float acc = 0.f;
    if (grp < groups) {
        const float *cs = ws.cs + (size_t)bh * L, *ds = ws.ds + (size_t)bh * L * 2;
#pragma unroll 4
        for (int i = grp; i < L; i += groups) {
            acc = __builtin_fmaf(cs[i], (float)kr[((size_t)b * L + i) * HF + (size_t)h * F + f], acc);
            acc = __builtin_fmaf(ds[2 * i], (float)q[((size_t)b * L + i) * HF + (size_t)h * F + f], acc);
        }
    }
    s_part[tid] = acc;
    __syncthreads();
    if (tid < F) {
        float sum = ws.row0[(size_t)bh * F + f] + ws.ds[(size_t)bh * L * 2 + 1] * (float)q[(size_t)b * L * HF + (size_t)h * F + f];
        for (int g = 0; g < groups; g++) sum += s_part[g * F + f];
        dkl[(size_t)b * L * HF + (size_t)h * F + f] = (T)sum;
    }
}

template <int NCH>
constexpr size_t bwd_parents_lds_bytes() {
    return (size_t)4 * bwd_wave_chunks<NCH, 3>() * 16 + sizeof(float) * (2 * ENT_FLOATS + 4 * 64);
}
template <int NCH>
constexpr size_t bwd_children_lds_bytes() {
    return (size_t)4 * bwd_wave_chunks<NCH, 2>() * 16 + sizeof(float) * (2 * ENT_FLOATS + 4 * (2 * PT * BWD_TD_PITCH + PT));
}
static_assert(bwd_parents_lds_bytes<8>() <= 160 * 1024 && bwd_children_lds_bytes<8>() <= 160 * 1024, "LDS of the backward kernels");

template <typename T, int NCH>
int launch_fused_bwd(const void *q, const void *kl, const void *kr, const float *gate, const float *lse, const float *links, const float *G,
                     const unsigned *masks, void *dq, void *dkl, void *dkr, float *dgate, float *wsp, int64_t B, int64_t L, int64_t H,
                     hipStream_t s) {
    constexpr int F = 2 * NCH * Chunk<T>::EPC;
    const size_t lds_p = bwd_parents_lds_bytes<NCH>(), lds_c = bwd_children_lds_bytes<NCH>();
    const BwdWorkspace ws = bwd_workspace(wsp, B, L, H, F);
    const unsigned tiles = (unsigned)((L + PT - 1) / PT), groups = (unsigned)((H + 3) / 4);
    const float scale = 1.0f / sqrtf((float)F);
    auto kp = links_fused_bwd_parents_kernel<T, NCH>;
    PCFGNAT_DYNAMIC_LDS(kp, lds_p);
    hipLaunchKernelGGL(kp, dim3(tiles, groups, (unsigned)B), dim3(LF_NT), lds_p, s, (const T *)q, (const T *)kl, (const T *)kr, gate, lse, links, G,
                       masks, (T *)dq, (T *)dkl, dgate, ws, (int)L, (int)H, scale * LF_LOG2E, scale);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    auto kc = links_fused_bwd_children_kernel<T, NCH>;
    PCFGNAT_DYNAMIC_LDS(kc, lds_c);
    hipLaunchKernelGGL(kc, dim3(tiles, groups, (unsigned)B), dim3(LF_NT), lds_c, s, (const T *)q, (const T *)kl, (const T *)kr, lse, links, G, masks,
                       (T *)dkr, ws, (int)L, (int)H, scale * LF_LOG2E, scale);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL((links_fused_bwd_row0_kernel<T>), dim3((unsigned)(B * H)), dim3(256), 0, s, (const T *)q, (const T *)kr, (T *)dkl, ws,
                       (int)L, (int)H, F);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

// the backward keeps two accumulator sets of F / 32 tiles per wave: head dimensions up to 64
bool fused_bwd_built(int dtype, int64_t F) { return fused_head_dim_built(dtype, F) && F <= 64; }

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

extern "C" int pcfgnat_extract_links_fused_backward_supported(int dtype, int64_t L, int64_t H, int64_t F) {
    if (!(H == 1 || H == 2 || H == 4 || H == 8 || H == 16) || L < 2 || L > 8192) return 0;
    return ((dtype == PCFGNAT_F16 || dtype == PCFGNAT_F32) && fused_bwd_built(dtype, F)) ? 1 : 0;
}

extern "C" size_t pcfgnat_extract_links_fused_backward_workspace_bytes(int64_t B, int64_t L, int64_t H, int64_t F) {
    if (B < 0 || L < 2 || H < 1 || F < 1) return 0;
    return bwd_workspace_words(B, L, H, F) * sizeof(float);
}

extern "C" int pcfgnat_extract_links_fused_backward(const float *grad_links, const float *links, const float *head_lse,
                                                    const unsigned *tile_masks, const void *query_chunks, const void *key_chunks_left,
                                                    const void *key_chunks_right, int dtype, const float *gate_logits, void *dq, void *dkl,
                                                    void *dkr, float *dgate, float *workspace, int64_t B, int64_t L, int64_t H, int64_t F,
                                                    void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 2 && F >= 1, "extract_links_fused_backward: bad dimensions (B=%lld L=%lld F=%lld)", (long long)B,
                    (long long)L, (long long)F);
    if (!pcfgnat_extract_links_fused_backward_supported(dtype, L, H, F))
        return fail(PCFGNAT_EUNSUPPORTED, "extract_links_fused_backward: dtype code %d, L = %lld, %lld heads of %lld is not built", dtype,
                    (long long)L, (long long)H, (long long)F);
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(grad_links && links && head_lse && tile_masks && query_chunks && key_chunks_left && key_chunks_right && gate_logits &&
                        dq && dkl && dkr && dgate && workspace,
                    "extract_links_fused_backward: null pointer");
    PCFGNAT_REQUIRE((((uintptr_t)query_chunks | (uintptr_t)key_chunks_left | (uintptr_t)key_chunks_right | (uintptr_t)links |
                      (uintptr_t)grad_links) & 15) == 0,
                    "extract_links_fused_backward: chunks, links and grad_links must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int nch = (int)(F / (dtype == PCFGNAT_F16 ? 16 : 8));
#define PCFGNAT_FUSED_BWD(T, n)                                                                                                     \
    return launch_fused_bwd<T, n>(query_chunks, key_chunks_left, key_chunks_right, gate_logits, head_lse, links, grad_links, tile_masks, \
                                  dq, dkl, dkr, dgate, workspace, B, L, H, s)
    if (dtype == PCFGNAT_F16) {
        if (nch == 1) PCFGNAT_FUSED_BWD(__half, 1);
        if (nch == 2) PCFGNAT_FUSED_BWD(__half, 2);
        PCFGNAT_FUSED_BWD(__half, 4);
    }
    if (nch == 1) PCFGNAT_FUSED_BWD(float, 1);
    if (nch == 2) PCFGNAT_FUSED_BWD(float, 2);
    if (nch == 4) PCFGNAT_FUSED_BWD(float, 4);
    PCFGNAT_FUSED_BWD(float, 8);
#undef PCFGNAT_FUSED_BWD
}
