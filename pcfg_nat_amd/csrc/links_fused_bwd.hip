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
//   dg:       one wave per (sentence, head, tile of 32 parents) runs over the tiles of right children and leaves dg, d gate;
//   main:     the same waves run over them again for dz and leave d q, d kl (all rows but row 0) and ds, while, in the
//             same launch, one wave per (sentence, head, tile of 32 right children) runs over the tiles of parents and
//             leaves d kr and the column sums of dz[.,0,.] (the two kinds of workgroups do not depend on each other and
//             fill the device together);
//   row 0:    d kl[0,h] from what the main launch left.
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
// log2 of the gate of head h from the row of gate logits (H <= 16; every load of the row in flight together)
__device__ __forceinline__ float log2_gate(const float *__restrict__ grow, int H, int h) {
    float gv[16], mx = NEG_INF_F, mine = 0.f;
#pragma unroll
    for (int j = 0; j < 16; j++) gv[j] = (j < H) ? grow[j] : NEG_INF_F;
#pragma unroll
    for (int j = 0; j < 16; j++) {
        mx = fmaxf(mx, gv[j]);
        mine = (j == h) ? gv[j] : mine;
    }
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 16; j++) sum += ex2((gv[j] - mx) * LF_LOG2E);
    return (mine - mx) * LF_LOG2E - lg2(sum);
}
__device__ __forceinline__ void lse_terms(float lse, ParentTerms &pt) {
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

// ---- fp16 chunks: the products with dz on the fp16 matrix instruction.  A value x S (S a power of two that brings the
// largest |x| of the tile just below 2^14) is handed over as the sum of two fp16 numbers, hi = x S rounded toward zero
// and lo = the rest, exact up to 2^-20 |x S| (2^-25 absolutely); the keys are fp16 already, so each product is two
// instructions of 16 contraction steps instead of sixteen fp32 instructions of two.
__device__ __forceinline__ void split_pair(float x0, float x1, float S, unsigned &hi, unsigned &lo) {
    const float y0 = x0 * S, y1 = x1 * S;
    const auto h = __builtin_amdgcn_cvt_pkrtz(y0, y1);
    hi = __builtin_bit_cast(unsigned, h);
    lo = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(y0 - (float)h[0], y1 - (float)h[1]));
}
// the lane's entries r = 8m .. 8m+7 as the operand of step m
__device__ __forceinline__ void split_operands(const float (&x)[16], float S, uint4 (&hi)[2], uint4 (&lo)[2]) {
#pragma unroll
    for (int m = 0; m < 2; m++) {
        split_pair(x[8 * m + 0], x[8 * m + 1], S, hi[m].x, lo[m].x);
        split_pair(x[8 * m + 2], x[8 * m + 3], S, hi[m].y, lo[m].y);
        split_pair(x[8 * m + 4], x[8 * m + 5], S, hi[m].z, lo[m].z);
        split_pair(x[8 * m + 6], x[8 * m + 7], S, hi[m].w, lo[m].w);
    }
}
// S and 1 / S for a tile whose largest magnitude over the wave is mx; false: nothing to add (all zero, or too small to matter)
__device__ __forceinline__ bool tile_scale(float mx, float &S, float &inv) {
    const int e = ((__float_as_int(mx) >> 23) & 255) - 127;  // floor(log2(mx)) for normal numbers
    if (!(mx > 0.f) || e < -100) return false;
    const int es = e > 100 ? 100 : e;  // (beyond that the values are not finite in any useful sense)
    S = __int_as_float((127 + 13 - es) << 23);
    inv = __int_as_float((127 - 13 + es) << 23);
    return true;
}
__device__ __forceinline__ floatx16 mma16(const uint4 &a, const uint4 &b, floatx16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), acc, 0, 0, 0);
}
__device__ __forceinline__ unsigned short half_bits(const uint4 &c, int i) {
    const unsigned w = (i < 2) ? c.x : (i < 4) ? c.y : (i < 6) ? c.z : c.w;
    return (unsigned short)(w >> (16 * (i & 1)));
}
// The tables in LDS are written and read through pointers of different types by the same wave (whose LDS operations
// execute in order): this keeps the compiler from moving the reads above the writes.
__device__ __forceinline__ void lds_order() { __asm__ volatile("" ::: "memory"); }
constexpr int KT_PITCH = 36;  // halves per row of a transposed tile [element][32 rows]: 8-byte reads of 32 lanes fall into 64 banks

// LDS per wave, in chunks: TILES tiles of 32 rows of one head (row pitch: the row plus one chunk) and one more row.
template <int NCH, int TILES>
constexpr int bwd_wave_chunks() {
    return TILES * PT * (2 * NCH + 1) + (2 * NCH + 1);
}
constexpr int BWD_TD_PITCH = 33;  // floats per row of a transposed 32 x 32 tile
constexpr int DH_PITCH = 40;      // halves per row of a [right child][parent] plane: 16-byte reads of 16 lanes fall into 64 banks
constexpr int BWD_TD_FLOATS = 4 * PT * DH_PITCH / 2;  // per wave: four fp16 planes, or two fp32 tiles and a row (fewer)
static_assert(BWD_TD_FLOATS >= 2 * PT * BWD_TD_PITCH + PT, "transposed tiles of the children's launch");

// ---- the parents' part of a workgroup: a tile of 32 parents, a group of four heads, sentence b;
// wave w takes head 4 * group + w (a wave without a head still helps to move the entries).  masks: [B,L,1+nw] words as
// the forward left them (flags, then the allowed right children).  MODE 0: the run that gives dg (and d gate); MODE 1:
// the run that gives dz and its products, with dg read back.
template <typename T, int NCH, int MODE>
__device__ __forceinline__ void bwd_parents(uint4 *lb_lds, int tile, int group, int b, const T *__restrict__ q, const T *__restrict__ kl,
                                            const T *__restrict__ kr,
                                            const float *__restrict__ gate, const float *__restrict__ head_lse,
                                            const float *__restrict__ links, const float *__restrict__ G, const unsigned *__restrict__ masks,
                                            T *__restrict__ dq, T *__restrict__ dkl, float *__restrict__ dgate, BwdWorkspace ws, int L, int H,
                                            float scale2, float scale) {
    constexpr int EPC = Chunk<T>::EPC, F = 2 * NCH * EPC, FT = (F + 31) / 32, RPC = 2 * NCH + 1;
    const int nw = (L + 31) / 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int a0 = tile * PT, h = group * 4 + wave;
    const bool active = h < H;
    constexpr int TILES = MODE == 0 ? 2 : 3;  // the run for dg keeps no table of the right keys
    uint4 *tQ = lb_lds + wave * bwd_wave_chunks<NCH, TILES>(), *tK1 = tQ + PT * RPC, *tKr = tK1 + PT * RPC, *tK0 = tQ + TILES * PT * RPC;
    float *s_ent = reinterpret_cast<float *>(lb_lds + 4 * bwd_wave_chunks<NCH, TILES>());  // two buffers of entries
    float *s_ds = s_ent + 2 * ENT_FLOATS + wave * 64;                                 // [2][32] per wave
    const int p = lane & 31, kb = lane >> 5, a = a0 + p;
    const bool in = a < L;
    const int ai = in ? a : 0, hh = active ? h : 0;
    const int HF = H * F;
    const bool vec4 = (L & 3) == 0;
    const unsigned *mrow = masks + ((size_t)b * L + ai) * (1 + nw);
    const unsigned flags = in ? mrow[0] : 1u;
    // The tiles of right children that hold an allowed (parent, right child) pair: [s_lo, s_hi).  The tiles in front of
    // the parents' own and those of the pad nodes behind the sentence hold none, contribute nothing and are not even
    // loaded (a step costs a trip to memory whatever it computes).  Masks do not depend on the head: every wave of the
    // workgroup finds the same range.
    // The first of them is requested on a guess, beside the masks: the parents' own tile, which is where the rules of a
    // parent begin (right children come behind their parent); a wrong guess costs the request a second time.
    const int guess = min(tile, nw - 1);
    EntryLoad ent;
    entries_request(links, G, b, a0, 32 * guess, L, vec4, tid, ent);
    int s_lo = nw, s_hi = 0;
    for (int ct = 0; ct < nw; ct++) {
        if (__ballot(in && (flags & 1u) == 0 && mrow[1 + ct] != 0u) != 0ull) {
            s_lo = min(s_lo, ct);
            s_hi = ct + 1;
        }
    }
    if (s_hi == 0) s_lo = guess;
    if (s_lo != guess) entries_request(links, G, b, a0, 32 * s_lo, L, vec4, tid, ent);  // (uniform over the workgroup)
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
        pt.lg2v = MODE == 0 ? log2_gate(gate + ((size_t)b * L + ai) * H, H, hh) : ws.lg[((size_t)b * L + ai) * H + hh];
        lse_terms(lse, pt);
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
    float dg = (MODE == 1 && in) ? ws.dg[((size_t)b * L + a) * H + hh] : 0.f, gsum = 0.f, ds0 = 0.f, ds1 = 0.f;
    uint4 cur[NCH], nxt[NCH];
    unsigned allow_cur, allow_nxt;
    right_keys(s_lo, cur, allow_cur);
    entries_store(s_ent, tid, ent);
    __syncthreads();
    // ---- one run over the tiles of right children: dg = sum G w (and the sum of G over the finite links), or dz and its
    // products with the right keys
#pragma unroll 1
    for (int s = s_lo; s < s_hi; s++) {
        const int ctn = min(s + 1, s_hi - 1);
        entries_request(links, G, b, a0, 32 * ctn, L, vec4, tid, ent);
        right_keys(ctn, nxt, allow_nxt);
        const float *buf = s_ent + ((s - s_lo) & 1) * ENT_FLOATS;
        // a tile without a single allowed (parent, right child) pair - the children in front of the parents, the pad nodes
        // behind the sentence - holds no finite link and contributes nothing: left out (the decision is the wave's)
        const bool live = __ballot(usable && allow_cur != 0u) != 0ull;
        if (active && live) {
            float g0[16], g1[16], l0[16], l1[16], z0[16], z1[16], dz0[16], dz1[16];
            entries_read(buf, 0, p, 0, kb, l0);
            entries_read(buf, 0, p, 1, kb, l1);
            entries_read(buf, 1, p, 0, kb, g0);
            entries_read(buf, 1, p, 1, kb, g1);
            scores(cur, allow_cur, z0, z1);
            if (MODE == 0) {
                entry_gradients<true>(z0, z1, g0, g1, l0, l1, pt, 0.f, scale, dg, gsum, dz0, dz1);
            } else {
                // the right keys of the tile as a table for the products below: [row][element], for fp16 [element][row]
                if constexpr (sizeof(T) == 2) {
                    unsigned short *krt = reinterpret_cast<unsigned short *>(tKr);
#pragma unroll
                    for (int j = 0; j < NCH; j++)
#pragma unroll
                        for (int i = 0; i < 8; i++) krt[((2 * j + kb) * 8 + i) * KT_PITCH + p] = half_bits(cur[j], i);
                } else {
#pragma unroll
                    for (int j = 0; j < NCH; j++) tKr[p * RPC + 2 * j + kb] = cur[j];
                }
                float unused_dg = 0.f, unused_gs = 0.f;
                entry_gradients<false>(z0, z1, g0, g1, l0, l1, pt, dg, scale, unused_dg, unused_gs, dz0, dz1);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    ds0 += dz0[r];
                    ds1 += dz1[r];
                }
                // d q[p][f] += sum_c (dz0 + dz1)[p][c] kr[c][f],  d kl[src(p)][f] += sum_c dz1[p][c] kr[c][f]: dz is already
                // laid out as the row operand (lane: parent p, right children acc_row(r, kb)); lane (f, kb) supplies the keys
                // of the same right children
                lds_order();
                if constexpr (sizeof(T) == 2) {
                    float dzs[16], mx = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        dzs[r] = dz0[r] + dz1[r];
                        mx = fmaxf(mx, fmaxf(fabsf(dzs[r]), fabsf(dz1[r])));
                    }
                    float S, inv;
                    if (tile_scale(wave_max(mx), S, inv)) {  // uniform
                        uint4 hs[2], ls[2], h1[2], l1[2];
                        split_operands(dzs, S, hs, ls);
                        split_operands(dz1, S, h1, l1);
                        const unsigned short *krt = reinterpret_cast<const unsigned short *>(tKr);
#pragma unroll
                        for (int t = 0; t < FT; t++) {
                            const int f = 32 * t + p;
                            floatx16 tq, tk;
#pragma unroll
                            for (int r = 0; r < 16; r++) tq[r] = tk[r] = 0.f;
#pragma unroll
                            for (int m = 0; m < 2; m++) {  // the right children acc_row(8m .. 8m+7, kb): 16m + 4kb + {0..3, 8..11}
                                uint4 bop = make_uint4(0, 0, 0, 0);
                                if (f < F) {
                                    const uint2 lo8 = *reinterpret_cast<const uint2 *>(krt + f * KT_PITCH + 16 * m + 4 * kb);
                                    const uint2 hi8 = *reinterpret_cast<const uint2 *>(krt + f * KT_PITCH + 16 * m + 8 + 4 * kb);
                                    bop = make_uint4(lo8.x, lo8.y, hi8.x, hi8.y);
                                }
                                tq = mma16(hs[m], bop, tq);
                                tk = mma16(h1[m], bop, tk);
                                tq = mma16(ls[m], bop, tq);
                                tk = mma16(l1[m], bop, tk);
                            }
#pragma unroll
                            for (int r = 0; r < 16; r++) {
                                accQ[t][r] = __builtin_fmaf(tq[r], inv, accQ[t][r]);
                                accK[t][r] = __builtin_fmaf(tk[r], inv, accK[t][r]);
                            }
                        }
                    }
                } else {
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
        }
#pragma unroll
        for (int j = 0; j < NCH; j++) cur[j] = nxt[j];
        allow_cur = allow_nxt;
        entries_store(s_ent + ((s - s_lo + 1) & 1) * ENT_FLOATS, tid, ent);
        __syncthreads();
    }
    if (MODE == 0 && active) {
        dg += __shfl_xor(dg, 32);
        gsum += __shfl_xor(gsum, 32);
        if (in && kb == 0) {
            // (the sum over the heads of dg is the sum of G over the finite links; a single head has a constant gate)
            dgate[((size_t)b * L + a) * H + h] = H == 1 ? 0.f : dg - ex2(pt.lg2v) * gsum;
            ws.dg[((size_t)b * L + a) * H + h] = dg;
            ws.lg[((size_t)b * L + a) * H + h] = pt.lg2v;
        }
    }
    if (!active || MODE == 0) return;
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
    lds_order();
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
            const float dk = accK[t][r] + (ar >= 1 ? d1[r] * qf[r] : 0.f);
            const int src = (ar - 1 < 0) ? L - 1 : ar - 1;
            if (ar < L) {
                dq[((size_t)b * L + ar) * HF + (size_t)h * F + f] = Chunk<T>::cast(accQ[t][r] + d0[r] * k0f + d1[r] * (ar == 0 ? k0f : k1f[r]));
                dkl[((size_t)b * L + src) * HF + (size_t)h * F + f] = Chunk<T>::cast(dk);  // (row 0 is written again by the last launch)
            }
            if (a0 == 0 && acc_row(r, kb) == 1) ws.row0[((size_t)b * H + h) * F + f] = dk;  // parent 1: row 0 as far as it gets here
        }
    }
}

// ---- the children's part of a workgroup: blockIdx.x = tile of 32 right children, blockIdx.y = group of four heads,
// sentence b; wave w takes head 4 * group + w.
template <typename T, int NCH>
__device__ __forceinline__ void bwd_children(uint4 *lb_lds, int tile, int group, int b, const T *__restrict__ q, const T *__restrict__ kl,
                                             const T *__restrict__ kr,
                                             const float *__restrict__ head_lse, const float *__restrict__ links,
                                             const float *__restrict__ G, const unsigned *__restrict__ masks, T *__restrict__ dkr,
                                             BwdWorkspace ws, int L, int H, float scale2, float scale) {
    constexpr int EPC = Chunk<T>::EPC, F = 2 * NCH * EPC, FT = (F + 31) / 32, RPC = 2 * NCH + 1;
    const int nw = (L + 31) / 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ct = tile, c0 = ct * PT, h = group * 4 + wave;
    const bool active = h < H;
    const int hh = active ? h : 0;
    uint4 *tQ = lb_lds + wave * bwd_wave_chunks<NCH, 2>(), *tK1 = tQ + PT * RPC, *tK0 = tK1 + PT * RPC;
    float *s_ent = reinterpret_cast<float *>(lb_lds + 4 * bwd_wave_chunks<NCH, 2>());
    float *tD = s_ent + 2 * ENT_FLOATS + wave * BWD_TD_FLOATS;  // fp32: [2][32][33], [32]; fp16: four planes
    float *s_cs = tD + 2 * PT * BWD_TD_PITCH;
    const int p = lane & 31, kb = lane >> 5;
    const int HF = H * F;
    const bool vec4 = (L & 3) == 0;
    // the tiles of parents that hold an allowed pair with this tile of right children: [p_lo, p_hi), as in the parents' part
    // (the first tile requested on a guess, tile 0: parents come in front of their right children)
    EntryLoad ent;
    entries_request(links, G, b, 0, c0, L, vec4, tid, ent);
    int p_lo = nw, p_hi = 0;
    for (int t = 0; t < nw; t++) {
        const int a = 32 * t + p;
        const unsigned *mrow = masks + ((size_t)b * L + min(a, L - 1)) * (1 + nw);
        if (__ballot(a < L && (mrow[0] & 1u) == 0 && mrow[1 + ct] != 0u) != 0ull) {
            p_lo = min(p_lo, t);
            p_hi = t + 1;
        }
    }
    if (p_hi == 0) p_lo = 0;
    if (p_lo != 0) entries_request(links, G, b, 32 * p_lo, c0, L, vec4, tid, ent);  // (the guess was tile 0; uniform over the workgroup)
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
    float cs0 = 0.f, csum[16];
#pragma unroll
    for (int r = 0; r < 16; r++) csum[r] = 0.f;
    ParentLoad cur, nxt;
    parent_request(p_lo, cur);
    entries_store(s_ent, tid, ent);
    __syncthreads();
#pragma unroll 1
    for (int pt = p_lo; pt < p_hi; pt++) {
        const int ptn = min(pt + 1, p_hi - 1);
        entries_request(links, G, b, 32 * ptn, c0, L, vec4, tid, ent);
        parent_request(ptn, nxt);
        const float *buf = s_ent + ((pt - p_lo) & 1) * ENT_FLOATS;
        // (a tile without an allowed pair contributes nothing, as in the parents' part)
        const bool live = __ballot((cur.flags & 1u) == 0 && cur.allow != 0u) != 0ull;
        if (active && live) {
            const int a = 32 * pt + p;
            ParentTerms ptm;
            ptm.lg2v = cur.lgv;
            lse_terms(cur.lse, ptm);
            // the parents' rows as chunks (column operand of the scores) and as tables for the products
            float sab0 = 0.f, sab1 = 0.f;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                if constexpr (sizeof(T) == 2) {  // [element][parent]
                    unsigned short *qt = reinterpret_cast<unsigned short *>(tQ), *k1t = reinterpret_cast<unsigned short *>(tK1);
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        qt[((2 * j + kb) * 8 + i) * KT_PITCH + p] = half_bits(cur.vq[j], i);
                        k1t[((2 * j + kb) * 8 + i) * KT_PITCH + p] = half_bits(cur.vk[j], i);
                    }
                } else {  // [parent][element]
                    tQ[p * RPC + 2 * j + kb] = cur.vq[j];
                    tK1[p * RPC + 2 * j + kb] = cur.vk[j];
                }
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
            // d kr[c][f] += sum_p (dz0 + dz1)[p][c] q[p][f] + sum_p dz1[p][c] kl[src(p)][f], and the column sums of dz0: dz goes
            // through LDS to the lanes of its right child (the row of the operand), lane (f, kb) supplies the parents' rows
            if constexpr (sizeof(T) == 2) {
                float dzs[16], mx = 0.f;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    dzs[r] = dz0[r] + dz1[r];
                    mx = fmaxf(mx, fmaxf(fabsf(dzs[r]), fabsf(dz1[r])));
                }
                float S, inv;
                if (tile_scale(wave_max(mx), S, inv)) {  // uniform
                    // four planes [right child][parent] of fp16: dz0 + dz1 as hi and lo, dz1 as hi and lo
                    unsigned short *dh = reinterpret_cast<unsigned short *>(tD);
#pragma unroll
                    for (int r = 0; r < 16; r += 2) {
                        unsigned hs, ls, h1, l1;
                        split_pair(dzs[r], dzs[r + 1], S, hs, ls);
                        split_pair(dz1[r], dz1[r + 1], S, h1, l1);
                        const int c_a = acc_row(r, kb) * DH_PITCH + p, c_b = acc_row(r + 1, kb) * DH_PITCH + p;
                        dh[0 * PT * DH_PITCH + c_a] = (unsigned short)hs;
                        dh[0 * PT * DH_PITCH + c_b] = (unsigned short)(hs >> 16);
                        dh[1 * PT * DH_PITCH + c_a] = (unsigned short)ls;
                        dh[1 * PT * DH_PITCH + c_b] = (unsigned short)(ls >> 16);
                        dh[2 * PT * DH_PITCH + c_a] = (unsigned short)h1;
                        dh[2 * PT * DH_PITCH + c_b] = (unsigned short)(h1 >> 16);
                        dh[3 * PT * DH_PITCH + c_a] = (unsigned short)l1;
                        dh[3 * PT * DH_PITCH + c_b] = (unsigned short)(l1 >> 16);
                    }
                    lds_order();
                    // step m: the parents 16m + 8kb .. + 7
                    uint4 aop[4][2];
#pragma unroll
                    for (int pl = 0; pl < 4; pl++)
#pragma unroll
                        for (int m = 0; m < 2; m++)
                            aop[pl][m] = *reinterpret_cast<const uint4 *>(dh + pl * PT * DH_PITCH + p * DH_PITCH + 16 * m + 8 * kb);
                    const unsigned short *qt = reinterpret_cast<const unsigned short *>(tQ), *k1t = reinterpret_cast<const unsigned short *>(tK1);
#pragma unroll
                    for (int t = 0; t < FT; t++) {
                        const int f = 32 * t + p;
                        floatx16 tr;
#pragma unroll
                        for (int r = 0; r < 16; r++) tr[r] = 0.f;
#pragma unroll
                        for (int m = 0; m < 2; m++) {
                            uint4 bq = make_uint4(0, 0, 0, 0), bk = bq;
                            if (f < F) {
                                const uint2 q0 = *reinterpret_cast<const uint2 *>(qt + f * KT_PITCH + 16 * m + 8 * kb);
                                const uint2 q1 = *reinterpret_cast<const uint2 *>(qt + f * KT_PITCH + 16 * m + 8 * kb + 4);
                                const uint2 k0 = *reinterpret_cast<const uint2 *>(k1t + f * KT_PITCH + 16 * m + 8 * kb);
                                const uint2 k1 = *reinterpret_cast<const uint2 *>(k1t + f * KT_PITCH + 16 * m + 8 * kb + 4);
                                bq = make_uint4(q0.x, q0.y, q1.x, q1.y);
                                bk = make_uint4(k0.x, k0.y, k1.x, k1.y);
                            }
                            tr = mma16(aop[0][m], bq, tr);
                            tr = mma16(aop[2][m], bk, tr);
                            tr = mma16(aop[1][m], bq, tr);
                            tr = mma16(aop[3][m], bk, tr);
                        }
#pragma unroll
                        for (int r = 0; r < 16; r++) accR[t][r] = __builtin_fmaf(tr[r], inv, accR[t][r]);
                    }
                    // the column sums of dz0 = (dz0 + dz1) - dz1: a product with a column of ones (every column of the result)
                    floatx16 tc;
#pragma unroll
                    for (int r = 0; r < 16; r++) tc[r] = 0.f;
                    const uint4 ones = make_uint4(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u);
#pragma unroll
                    for (int m = 0; m < 2; m++) {
                        const uint4 n1 = make_uint4(aop[2][m].x ^ 0x80008000u, aop[2][m].y ^ 0x80008000u, aop[2][m].z ^ 0x80008000u,
                                                    aop[2][m].w ^ 0x80008000u);
                        const uint4 n3 = make_uint4(aop[3][m].x ^ 0x80008000u, aop[3][m].y ^ 0x80008000u, aop[3][m].z ^ 0x80008000u,
                                                    aop[3][m].w ^ 0x80008000u);
                        tc = mma16(aop[0][m], ones, tc);
                        tc = mma16(n1, ones, tc);
                        tc = mma16(aop[1][m], ones, tc);
                        tc = mma16(n3, ones, tc);
                    }
#pragma unroll
                    for (int r = 0; r < 16; r++) csum[r] = __builtin_fmaf(tc[r], inv, csum[r]);
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    tD[p * BWD_TD_PITCH + acc_row(r, kb)] = dz0[r];
                    tD[(PT + p) * BWD_TD_PITCH + acc_row(r, kb)] = dz1[r];
                }
                lds_order();
                // lane (c, kb) supplies the gradients of parent 2 s + kb in step s, lane (f, kb) the elements of that parent's rows
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
        }
        cur = nxt;
        entries_store(s_ent + ((pt - p_lo + 1) & 1) * ENT_FLOATS, tid, ent);
        __syncthreads();
    }
    if (!active) return;
    // ---- the column sums: per lane for the right children acc_row(r, kb) it stores below
    if constexpr (sizeof(T) == 2) {
        if (p == 0) {
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (c0 + acc_row(r, kb) < L) ws.cs[((size_t)b * H + h) * L + c0 + acc_row(r, kb)] = csum[r];
        }
    } else {
        cs0 += __shfl_xor(cs0, 32);  // lane (c, kb) summed the parents of its half
        if (kb == 0) {
            s_cs[p] = cs0;
            if (c0 + p < L) ws.cs[((size_t)b * H + h) * L + c0 + p] = cs0;
        }
#pragma unroll
        for (int r = 0; r < 16; r++) csum[r] = s_cs[acc_row(r, kb)];
    }
    lds_order();
    // ---- the null option's left key and the stores: lane (f, kb) holds the right children acc_row(r, kb) of column f
#pragma unroll
    for (int t = 0; t < FT; t++) {
        const int f = 32 * t + p;
        if (f >= F) continue;
        const float k0f = Chunk<T>::elem(tK0, f);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int c = c0 + acc_row(r, kb);
            if (c < L) dkr[((size_t)b * L + c) * HF + (size_t)h * F + f] = Chunk<T>::cast(accR[t][r] + csum[r] * k0f);
        }
    }
}

// ---- first launch: dg, d gate.  grid (tiles of 32 parents, groups of four heads, B)
template <typename T, int NCH>
__global__ __launch_bounds__(LF_NT) void links_fused_bwd_dg_kernel(const T *__restrict__ q, const T *__restrict__ kl, const T *__restrict__ kr,
                                                                  const float *__restrict__ gate, const float *__restrict__ head_lse,
                                                                  const float *__restrict__ links, const float *__restrict__ G,
                                                                  const unsigned *__restrict__ masks, float *__restrict__ dgate,
                                                                  BwdWorkspace ws, int L, int H, float scale2, float scale) {
    extern __shared__ uint4 lb_lds[];
    bwd_parents<T, NCH, 0>(lb_lds, blockIdx.x, blockIdx.y, blockIdx.z, q, kl, kr, gate, head_lse, links, G, masks, nullptr, nullptr, dgate, ws, L, H,
                           scale2, scale);
}

// ---- second launch: the parents' and the children's parts side by side, so that the device is filled by both.
// grid (tiles of 32, groups of four heads, 2 B): tiles x groups x B workgroups for the parents and as many for the children.
template <typename T, int NCH>
__global__ __launch_bounds__(LF_NT) void links_fused_bwd_main_kernel(const T *__restrict__ q, const T *__restrict__ kl, const T *__restrict__ kr,
                                                                    const float *__restrict__ gate, const float *__restrict__ head_lse,
                                                                    const float *__restrict__ links, const float *__restrict__ G,
                                                                    const unsigned *__restrict__ masks, T *__restrict__ dq, T *__restrict__ dkl,
                                                                    T *__restrict__ dkr, BwdWorkspace ws, int B, int L, int H, float scale2,
                                                                    float scale) {
    extern __shared__ uint4 lb_lds[];
    // Which (role, tile, group of heads, sentence) a workgroup takes follows from its place in the launch order (x runs
    // fastest), heaviest first: a tile of parents has the tiles of right children from its own on to do, a tile of right
    // children the tiles of parents up to its own, so the first tile of parents and the last of children lead, and the
    // workgroups that find most of their tiles masked come when the others are running out.
    const int tiles = gridDim.x, groups = gridDim.y;
    const int n = blockIdx.x + tiles * (blockIdx.y + groups * blockIdx.z), per_class = groups * 2 * B;
    const int k = n / per_class, j = n - k * per_class, role = j & 1, r = j >> 1, group = r % groups, b = r / groups;
    if (role == 0)
        bwd_parents<T, NCH, 1>(lb_lds, k, group, b, q, kl, kr, gate, head_lse, links, G, masks, dq, dkl, nullptr, ws, L, H, scale2, scale);
    else
        bwd_children<T, NCH>(lb_lds, tiles - 1 - k, group, b, q, kl, kr, head_lse, links, G, masks, dkr, ws, L, H, scale2, scale);
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
constexpr size_t bwd_dg_lds_bytes() {
    return (size_t)4 * bwd_wave_chunks<NCH, 2>() * 16 + sizeof(float) * (2 * ENT_FLOATS + 4 * 64);
}
template <int NCH>
constexpr size_t bwd_children_lds_bytes() {
    return (size_t)4 * bwd_wave_chunks<NCH, 2>() * 16 + sizeof(float) * (2 * ENT_FLOATS + 4 * BWD_TD_FLOATS);
}
static_assert(bwd_parents_lds_bytes<8>() <= 160 * 1024 && bwd_children_lds_bytes<8>() <= 160 * 1024, "LDS of the backward kernels");

template <typename T, int NCH>
int launch_fused_bwd(const void *q, const void *kl, const void *kr, const float *gate, const float *lse, const float *links, const float *G,
                     const unsigned *masks, void *dq, void *dkl, void *dkr, float *dgate, float *wsp, int64_t B, int64_t L, int64_t H,
                     hipStream_t s) {
    constexpr int F = 2 * NCH * Chunk<T>::EPC;
    const size_t lds_p = bwd_parents_lds_bytes<NCH>(), lds_c = bwd_children_lds_bytes<NCH>(), lds_m = lds_p > lds_c ? lds_p : lds_c;
    const BwdWorkspace ws = bwd_workspace(wsp, B, L, H, F);
    const unsigned tiles = (unsigned)((L + PT - 1) / PT), groups = (unsigned)((H + 3) / 4);
    const float scale = 1.0f / sqrtf((float)F);
    auto kd = links_fused_bwd_dg_kernel<T, NCH>;
    PCFGNAT_DYNAMIC_LDS(kd, bwd_dg_lds_bytes<NCH>());
    hipLaunchKernelGGL(kd, dim3(tiles, groups, (unsigned)B), dim3(LF_NT), bwd_dg_lds_bytes<NCH>(), s, (const T *)q, (const T *)kl, (const T *)kr, gate, lse, links, G,
                       masks, dgate, ws, (int)L, (int)H, scale * LF_LOG2E, scale);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    auto km = links_fused_bwd_main_kernel<T, NCH>;
    PCFGNAT_DYNAMIC_LDS(km, lds_m);
    hipLaunchKernelGGL(km, dim3(tiles, groups, (unsigned)(2 * B)), dim3(LF_NT), lds_m, s, (const T *)q, (const T *)kl, (const T *)kr, gate, lse, links,
                       G, masks, (T *)dq, (T *)dkl, (T *)dkr, ws, (int)B, (int)L, (int)H, scale * LF_LOG2E, scale);
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
    PCFGNAT_REQUIRE(B >= 0 && B <= 32767 && L >= 2 && F >= 1, "extract_links_fused_backward: bad dimensions (B=%lld L=%lld F=%lld)",
                    (long long)B, (long long)L, (long long)F);
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
