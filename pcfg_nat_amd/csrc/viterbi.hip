// Viterbi (max-product) tables per output length with back-pointers, and the tree-to-sequence readout.
//
// Replaces the reference's pcfg_viterbi.cu (calculate_C_kernel :177-241, calculate_S_kernel :22-140) and the
// host loop viterbi_decoding (pcfg_loss.cpp:12-73), for max_left = 1 - and for max_left = 3 where a sentence's links hold
// no rule of a composite local tree (viterbi_ml3_kernel; any other case: generic_ml.hip).
//
// S[a][len] = ob[a] + max over (c >= a, j in {0,1}) of links[a][j][c] + C[j] + S[c][len-j-1], with C[0] = 0 (null left
// child) and C[1] = ob[a-1] (the local leaf).  Every candidate is evaluated as ((links + C) + S) + ob in fp32, the
// reference's association order, so table values and arg-max decisions are reproducible bit for bit; exact ties
// follow the reference's 4-lane strided scan (lane priority 0 > 2 > 1 > 3, then c ascending, then j ascending).
//
// Same sweep shape as the inside forward: one workgroup per sentence, one 16-lane DPP row per parent node, link
// slabs in registers (graphs of up to 514 nodes), one barrier per length.
#include "common.hip.h"

namespace pcfgnat {
namespace {

constexpr int NT = 1024;

__device__ __forceinline__ int tie_key(int rel_c, int j) {
    const int lane = rel_c & 3;
    const int rank = (lane == 0) ? 0 : (lane == 2) ? 1 : (lane == 1) ? 2 : 3;
    return (rank << 24) | (rel_c << 1) | j;
}

__device__ __forceinline__ void take_better(float &best, int &key, float ov, int ok) {
    if (ov > best || (ov == best && ok < key)) {
        best = ov;
        key = ok;
    }
}

template <int CTRL>
__device__ __forceinline__ void row16_argmax_step(float &best, int &key) {
    const float ov = dpp_f<CTRL>(best);
    const int ok = dpp_i<CTRL>(key);
    take_better(best, key, ov, ok);
}

__device__ __forceinline__ float nan_to_ninf(float v) { return (v != v) ? NEG_INF_F : v; }

// Diagnostic: sentences whose pipelined sweep gave up and which the one-workgroup kernel therefore redid, since the library
// was loaded (pcfgnat_pipeline_redo_counts).
__device__ unsigned long long g_viterbi_redone;

// Row maximum with one DPP instruction per step; inputs are never NaN here.
__device__ __forceinline__ float row16_max_raw(float v) {
    return dpp_max_mirror(dpp_max_half_mirror(dpp_max_xor2(dpp_max_xor1(v))));
}

// Back-pointer accessors of the readout walk.  FullTraces: the reference's three int64 tables [L][Lq].
struct FullTraces {
    const int64_t *Li, *Ri, *Mi;
    int Lq;
    __host__ __device__ int64_t left(int64_t node, int64_t len) const { return Li[node * Lq + len]; }
    __host__ __device__ int64_t right(int64_t node, int64_t len) const { return Ri[node * Lq + len]; }
    __host__ __device__ int64_t mid(int64_t node, int64_t len) const { return Mi[node * Lq + len]; }
};
// What the walk reads besides the traces: the nodes' tokens and the left-tree mask, from memory.
struct WalkInputs {
    const int64_t *tok, *mask;
    int64_t mask_dim;
    __host__ __device__ bool in_range(int64_t node, int64_t l) const { return !(l < 0 || l >= mask_dim || node >= mask_dim); }
    __host__ __device__ bool forbidden(int64_t node, int64_t l) const { return mask[node * mask_dim + l] != 0; }
    __host__ __device__ int64_t token(int64_t node) const { return tok[node]; }
};

// One walk per sentence (pcfg_loss.cpp:22-59).  Shared by the device kernels and the host entry point.  SI = integer
// type of the explicit stacks.
template <typename Traces, typename Inputs, typename SI>
__host__ __device__ inline int64_t readout_one(int64_t pred_len, int64_t max_h, const Traces &tr, const Inputs &in, int64_t pad,
                                               int64_t *out, SI *stack_node, SI *stack_len, int L, int Lq) {
    const int cap = L;
    int sp = 0;
    int64_t cnt = 0, node = 1, len = pred_len, last = -1;
    if (len < 0 || len >= Lq) return -1;
    int64_t budget = (int64_t)L * Lq + L;  // well-formed traces visit each (node, len) cell at most once
    while ((node < max_h && node != 0) || sp > 0) {
        if (--budget < 0) return -1;
        while (node < max_h && node != 0) {
            if (sp >= cap || node < 0 || node >= L || len < 0 || len >= Lq) return -1;
            stack_node[sp] = (SI)node;
            stack_len[sp] = (SI)len;
            sp++;
            int64_t l = tr.left(node, len);
            l = (l == node) ? 0 : l;
            if (!in.in_range(node, l)) return -1;
            if (in.forbidden(node, l)) break;
            const int64_t nl = tr.mid(node, len);
            node = l;
            len = nl;
        }
        sp--;
        node = stack_node[sp];
        len = stack_len[sp];
        const int64_t t = in.token(node);
        if (t != pad && t != last) {
            last = t;
            if (cnt >= cap) return -1;
            out[cnt++] = t;
        }
        const int64_t r = tr.right(node, len);
        const int64_t nl = len - tr.mid(node, len) - 1;
        node = r;
        len = nl;
    }
    return cnt;
}

// The same walk over the compact records of the single-call decode (max_left = 1): one int32 per (main-chain node,
// length), 0 = empty cell, else 1 + ((c_id - a_id) << 1 | j); the rows of the local leaves are never written and read as
// zeros, as they do in the full tables.  With such traces the walk needs no stack: it runs down the main chain, and a
// node's left child is the null node or the leaf in front of it, whose own children are null - so per main-chain node
// the walk above emits the leaf (if the record names it, it is not node 0 and the mask allows the descent), then the
// node, and goes on to the right child with what is left of the length.  Inputs staged in LDS by the workgroup: the
// tokens, and of the mask the one entry per node that can matter, (node, node - 1).  W holds [rows][stride] records.
// Returns the number of tokens emitted, -1 for malformed traces (as readout_one).
__device__ inline int64_t walk_compact_ml1(int pred_len, int64_t max_h, const int *W, int stride, int rows, const int64_t *tok,
                                           const unsigned char *leaf_forbidden, int64_t mask_dim, int64_t pad, int64_t *out, int L,
                                           int Lq) {
    int64_t cnt = 0, last = -1;
    int node = 1, len = pred_len;
    if (len < 0 || len >= Lq) return -1;
    while (node < max_h && node != 0) {
        if (node >= L || len < 0 || len >= Lq || node >= mask_dim) return -1;
        const int a_id = node >> 1;
        const int r = ((node & 1) && a_id < rows) ? W[a_id * stride + len] : 0;
        const int j = (r != 0) ? ((r - 1) & 1) : 0;
        if (j && node > 1 && !leaf_forbidden[node]) {
            const int64_t t = tok[node - 1];
            if (t != pad && t != last) {
                last = t;
                if (cnt >= L) return -1;
                out[cnt++] = t;
            }
        }
        const int64_t t = tok[node];
        if (t != pad && t != last) {
            last = t;
            if (cnt >= L) return -1;
            out[cnt++] = t;
        }
        node = (r != 0) ? 2 * (a_id + ((r - 1) >> 1)) + 1 : 0;
        len = len - j - 1;
    }
    return cnt;
}

// Length selection (glat_decomposed_with_link_two_hands_tri_pcfg.py:489-497) by one wave: arg max over len >= 1 of
// scores[len] / penalty[len] with NaN read as -inf, first maximum wins; every lane returns the result.
__device__ __forceinline__ int select_length(const float *scores, const float *penalty, int Lq, int lane) {
    float best = NEG_INF_F;
    int idx = 0x7fffffff;
    for (int len = 1 + lane; len < Lq; len += 64) {
        float v = scores[len] / penalty[len];
        v = (v != v) ? NEG_INF_F : v;
        if (v > best) {
            best = v;
            idx = len;
        }
    }
    const float top = wave_max(best);
    const int cand = wave_min((best == top && idx != 0x7fffffff) ? idx : 0x7fffffff);
    return cand == 0x7fffffff ? 1 : cand;  // nothing above -inf: torch.max returns the first index
}

// NQ = number of 16-node chunks of the main chain (mc <= 16*NQ <= 256).  Row pass r handles parents 64r .. 64r+63, one
// 16-lane row per parent; its lanes stride over the children, of which only chunks q >= 4r can hold c >= a, so the
// triangular slabs cost NQ + (NQ-4) + (NQ-8) + ... chunk pairs of registers per thread.  Everything that does not
// change from length to length is folded into the slabs once (links + 0 and links + ob[leaf], in the reference's
// association order), which leaves two adds, one compare and two selects per candidate and length.  Inside a thread the
// candidates are visited in ascending (child, j) order and only a strictly larger value replaces the running best,
// which is the reference's tie order for one lane of its strided scan; the full tie key is built once per row and used
// in the cross-lane reduction.  LDS: three rotating columns (lengths len, len-1, len-2).
//
// COMPACT = false: the reference's outputs, S and the three int64 trace tables.  COMPACT = true (whole decode in one
// launch): the sweep only leaves one int32 per (main node, length) in a workspace and the root's scores in LDS; the
// same workgroup then selects the output length and walks the tree.
struct DecodeArgs {
    const int64_t *tokens, *mask;  // [B][L], [mask_dim][mask_dim]
    const float *penalty;          // [Lq]
    int *W;                        // [B][L/2][Lq] workspace
    int64_t *out_tokens, *out_count, *pred_length;
    float *out_tokens_f32;         // [B][L] or null: the emitted tokens once more as float32, the type the model hands on
    int64_t mask_dim, pad;
    // set when the pipelined sweep has run before this kernel: sentences whose flag is down only need the length
    // selection (root scores [B][Lq]) and the walk, the others are redone from scratch
    const int *pipe_flags;
    const float *pipe_scores;
};

template <int NQ, bool COMPACT>
__global__ __launch_bounds__(NT) void viterbi_ml1_kernel(const float *__restrict__ ob_lprob, const float *__restrict__ links,
                                                        const int64_t *__restrict__ out_len, float *__restrict__ S,
                                                        int64_t *__restrict__ Rt, int64_t *__restrict__ Lt, int64_t *__restrict__ Mt,
                                                        int L, int Lq, DecodeArgs dec) {
    constexpr int R = (NQ + 3) / 4;
    constexpr int MP = 64 * R;
    __shared__ float col[3 * MP];
    // COMPACT: tokens [L] (int64), scores [Lq] (float), mask entries [L] (bytes)
    extern __shared__ __align__(8) int64_t dyn64[];
    int64_t *sm_tok = dyn64;
    float *sm_scores = reinterpret_cast<float *>(dyn64 + L);
    unsigned char *sm_leaf = reinterpret_cast<unsigned char *>(sm_scores + Lq);
    const int b = blockIdx.x, tid = threadIdx.x, gidx = tid >> 4, j16 = tid & 15;
    const int m = (int)out_len[b];
    const float *ob = ob_lprob + (size_t)b * L;
    const float *lk = links + (size_t)b * L * 2 * L;
    const size_t tab = (size_t)b * L * Lq;
    float *Sb = S + tab;
    int64_t *Rb = Rt + tab, *Lb = Lt + tab, *Mb = Mt + tab;
    const int rowsW = L / 2;
    int *Wb = COMPACT ? dec.W + (size_t)b * rowsW * Lq : nullptr;
    const bool in_contract = !(m < 2 || m > L || (m % 2) != 0);
    const bool from_pipe = COMPACT && dec.pipe_flags != nullptr && dec.pipe_flags[b] == 0;  // workgroup-uniform
    if (COMPACT && dec.pipe_flags != nullptr && !from_pipe && tid == 0) atomicAdd(&g_viterbi_redone, 1ull);

    if (COMPACT) {
        if (!from_pipe)
            for (int i = tid; i < rowsW * Lq; i += NT) Wb[i] = 0;
        for (int i = tid; i < Lq; i += NT) sm_scores[i] = from_pipe ? dec.pipe_scores[(size_t)b * Lq + i] : NEG_INF_F;
        for (int i = tid; i < L; i += NT) {
            dec.out_tokens[(size_t)b * L + i] = dec.pad;
            // what the walk will read, staged while the sweep runs
            sm_tok[i] = dec.tokens[(size_t)b * L + i];
            sm_leaf[i] = (i < dec.mask_dim && i >= 1 && dec.mask[(size_t)i * dec.mask_dim + (i - 1)] != 0) ? 1 : 0;
        }
    } else {
        // tables start as -inf / 0 (pcfg_viterbi.cu:159, 287-289)
        for (size_t i = tid; i < (size_t)L * Lq; i += NT) {
            Sb[i] = NEG_INF_F;
            Rb[i] = 0;
            Lb[i] = 0;
            Mb[i] = 0;
        }
        if (!in_contract) return;  // out of contract: leave the empty tables
    }
    if (in_contract && !from_pipe) {
    const int mc = m / 2;

    // slabs: unconditional loads from clamped addresses (all in flight together), masked afterwards
    float A0[R][NQ], A1[R][NQ], ob_a[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a_id = gidx + 64 * r, a = 2 * min(a_id, mc - 1) + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q >= 4 * r) {
                const int c = 2 * min(j16 + 16 * q, mc - 1) + 1;
                A0[r][q] = lk[((size_t)a * 2 + 0) * L + c];
                A1[r][q] = lk[((size_t)a * 2 + 1) * L + c];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a_id = gidx + 64 * r, a = 2 * min(a_id, mc - 1) + 1;
        const float oa = ob[a], ol = ob[a - 1];
        ob_a[r] = (a_id < mc) ? oa : NEG_INF_F;
        const float ob_leaf = (a_id < mc && a_id >= 1) ? ol : NEG_INF_F;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q >= 4 * r) {
                const int c_id = j16 + 16 * q;
                const bool ok = a_id < mc && c_id < mc && c_id >= a_id;
                A0[r][q] = ok ? A0[r][q] + 0.f : NEG_INF_F;
                A1[r][q] = (ok && a_id >= 1) ? A1[r][q] + ob_leaf : NEG_INF_F;
            }
        }
    }
    // length 0: nothing; length 1: only the last node (pcfg_viterbi.cu:57-59)
    for (int i = tid; i < 3 * MP; i += NT) col[i] = (i == 1 * MP + mc - 1) ? ob[m - 1] : NEG_INF_F;
    __syncthreads();
    if (tid == 0 && Lq > 1) {
        if (COMPACT) {
            if (m - 1 == 1) sm_scores[1] = ob[m - 1];
        } else {
            Sb[(size_t)(m - 1) * Lq + 1] = ob[m - 1];
        }
    }

    const int len_end = m / 4;  // pcfg_viterbi.cu:67
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int i1 = 1, i2 = 0, i0 = 2;  // column slots of len-1, len-2, len
    for (int len = 2; len < len_end; len++) {
        const float *cur1 = col + i1 * MP, *cur2 = col + i2 * MP;
        float *nxt = col + i0 * MP;
        // the two columns stay in registers across the row passes, except for the widest slabs, which re-read them from
        // LDS in every pass to stay inside the register budget of a 1024-thread workgroup
        constexpr bool RELOAD = NQ > 12;
        float sc1[NQ], sc2[NQ];
        if (!RELOAD) {
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                sc1[q] = cur1[j16 + 16 * q];
                sc2[q] = cur2[j16 + 16 * q];
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int a_id = gidx + 64 * r;
            // The link matrices are triangular and the sentence may be shorter than the slabs: a wave whose four parents
            // all lie behind the last node has nothing to do in this pass, and a chunk of children that lies in front of
            // all four parents, or behind the last node, holds no candidate for it.  (Wave-uniform tests; the columns
            // keep their initial -inf in the rows nobody writes.)
            const int row_lo = 64 * r + 4 * wave;
            if (row_lo >= mc) continue;
            float best = NEG_INF_F;
            int sel = -1;
            if (RELOAD) {
                asm volatile("" ::: "memory");  // keeps the compiler from merging the passes' loads back into one set
#pragma unroll
                for (int q = 0; q < NQ; q++) {
                    if (q >= 4 * r) {
                        sc1[q] = cur1[j16 + 16 * q];
                        sc2[q] = cur2[j16 + 16 * q];
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q >= 4 * r && 16 * q + 15 >= row_lo && 16 * q < mc) {
                    const float c0 = (A0[r][q] + sc1[q]) + ob_a[r];
                    const float c1 = (A1[r][q] + sc2[q]) + ob_a[r];
                    if (c0 > best) {  // false for NaN and for -inf against the initial -inf
                        best = c0;
                        sel = 2 * q;
                    }
                    if (c1 > best) {
                        best = c1;
                        sel = 2 * q + 1;
                    }
                }
            }
            // row maximum first, then the smallest tie key among the lanes that hold it
            const float mine = best;
            best = row16_max_raw(best);
            int key = (sel < 0 || mine != best) ? 0x7fffffff : tie_key(j16 + 16 * (sel >> 1) - a_id, sel & 1);
            key = min(key, dpp_i<DPP_QUAD_XOR1>(key));
            key = min(key, dpp_i<DPP_QUAD_XOR2>(key));
            key = min(key, dpp_i<DPP_ROW_HALF_MIRROR>(key));
            key = min(key, dpp_i<DPP_ROW_MIRROR>(key));
            if (j16 == 0) {
                nxt[a_id] = best;
                if (best != NEG_INF_F && a_id < mc) {  // pcfg_viterbi.cu:125-131
                    const int a = 2 * a_id + 1;
                    const int jj = key & 1, rel = (key >> 1) & 0x7fffff;
                    if (COMPACT) {
                        Wb[(unsigned)(a_id * Lq + len)] = 1 + ((rel << 1) | jj);
                        if (a_id == 0) sm_scores[len] = best;
                    } else {
                        const unsigned o = (unsigned)(a * Lq + len);  // 32-bit offset from the uniform table bases
                        Sb[o] = best;
                        Lb[o] = jj ? (a - 1) : 0;
                        Rb[o] = 2 * (a_id + rel) + 1;
                        Mb[o] = jj;
                    }
                }
            }
        }
        const int t = i2;
        i2 = i1;
        i1 = i0;
        i0 = t;
        lds_barrier();
    }
    }  // in_contract
    if (COMPACT) {
        __syncthreads();  // the workspace records and the padded output row are visible to the walking thread
        int64_t count = 0;
        if (tid < 64) {
            const int pl = select_length(sm_scores, dec.penalty, Lq, tid);
            if (tid == 0) {
                dec.pred_length[b] = pl;
                count = walk_compact_ml1(pl, out_len[b], Wb, Lq, rowsW, sm_tok, sm_leaf, dec.mask_dim, dec.pad,
                                         dec.out_tokens + (size_t)b * L, L, Lq);
            }
        }
        if (dec.out_tokens_f32 != nullptr) {  // workgroup-uniform
            __syncthreads();                  // the walked row is visible to the whole workgroup
            for (int i = tid; i < L; i += NT) dec.out_tokens_f32[(size_t)b * L + i] = (float)dec.out_tokens[(size_t)b * L + i];
        }
        // the count goes out last: a host that watches it in pinned memory finds the sentence's kernel as good as through
        if (tid == 0) dec.out_count[b] = count;
    }
}

// ------------------------------------------------------------------------------------------------------------
// max_left = 3 (two layers of local tree in front of every main-chain node; pcfg_viterbi.cu:22-140 with ml = 3) for
// sentences whose links hold no rule of a composite local tree (ml3_composite_rules: every sentence the model's scorer can
// produce, where a local node has no allowed right child).  Then calculate_C_kernel (:177-241) leaves only the two leaves
// a-1 and a-3 with yield 1 and the null child with yield 0, and the main-chain recursion is the one above with a stride of
// four nodes and three left options per (parent, child) instead of two:
//   S[a][len] = ob[a] + max over c of  links[a][0][c] + 0 + S[c][len-1],  links[a][3][c] + ob[a-3] + S[c][len-2],
//                                      links[a][1][c] + ob[a-1] + S[c][len-2]
// visited in that order per child, which is the reference's (yield j ascending, then left node b ascending), with the
// same association order and the same tie order across its 4-lane strided scan.  Outputs are the reference's full tables.
// A sentence that does hold such a rule is left untouched for the general kernel launched behind (skip_ml3_taken).
__device__ unsigned long long g_viterbi_ml3_counts[2];  // diagnostic: sentences served here, sentences left to the general kernel

__device__ __forceinline__ int tie_key3(int rel_c, int option) {
    const int lane = rel_c & 3;
    const int rank = (lane == 0) ? 0 : (lane == 2) ? 1 : (lane == 1) ? 2 : 3;
    return (rank << 24) | (rel_c << 2) | option;
}

template <int NQ>
__global__ __launch_bounds__(NT) void viterbi_ml3_kernel(const float *__restrict__ ob_lprob, const float *__restrict__ links,
                                                        const int64_t *__restrict__ out_len, float *__restrict__ S,
                                                        int64_t *__restrict__ Rt, int64_t *__restrict__ Lt, int64_t *__restrict__ Mt,
                                                        int L, int Lq) {
    constexpr int R = (NQ + 3) / 4;
    constexpr int MP = 64 * R;
    __shared__ float col[3 * MP];
    const int b = blockIdx.x, tid = threadIdx.x, gidx = tid >> 4, j16 = tid & 15;
    const int m = (int)out_len[b];
    const float *ob = ob_lprob + (size_t)b * L;
    const float *lk = links + (size_t)b * L * 4 * L;
    const size_t tab = (size_t)b * L * Lq;
    float *Sb = S + tab;
    int64_t *Rb = Rt + tab, *Lb = Lt + tab, *Mb = Mt + tab;
    const bool in_contract = !(m < 2 || m > L || ((m - 2) % 4) != 0);
    const bool composite = in_contract && ml3_composite_rules<NT>(lk, L, m, tid);  // workgroup-uniform
    if (tid == 0) atomicAdd(&g_viterbi_ml3_counts[composite ? 1 : 0], 1ull);
    if (composite) return;
    for (size_t i = tid; i < (size_t)L * Lq; i += NT) {  // pcfg_viterbi.cu:159, 287-289
        Sb[i] = NEG_INF_F;
        Rb[i] = 0;
        Lb[i] = 0;
        Mb[i] = 0;
    }
    if (!in_contract) return;  // out of contract: the empty tables
    const int mc = (m - 2) / 4 + 1;

    // slabs: unconditional loads from clamped addresses (all in flight together), masked afterwards; what does not change
    // from length to length (links + 0, links + ob[leaf]) is added once, in the reference's association order
    float A0[R][NQ], A3[R][NQ], A1[R][NQ], ob_a[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a = 4 * min(gidx + 64 * r, mc - 1) + 1;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q >= 4 * r) {
                const int c = 4 * min(j16 + 16 * q, mc - 1) + 1;
                A0[r][q] = lk[((size_t)a * 4 + 0) * L + c];
                A3[r][q] = lk[((size_t)a * 4 + 3) * L + c];
                A1[r][q] = lk[((size_t)a * 4 + 1) * L + c];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int a_id = gidx + 64 * r, a = 4 * min(a_id, mc - 1) + 1;
        const float oa = ob[a], leaf1 = ob[a - 1], leaf3 = ob[max(a - 3, 0)];
        ob_a[r] = (a_id < mc) ? oa : NEG_INF_F;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            if (q >= 4 * r) {
                const int c_id = j16 + 16 * q;
                const bool ok = a_id < mc && c_id < mc && c_id >= a_id;
                const bool with_leaf = ok && a_id >= 1;  // the root's only left child is the null node (:70, b_start = 1)
                A0[r][q] = ok ? A0[r][q] + 0.f : NEG_INF_F;
                A3[r][q] = with_leaf ? A3[r][q] + leaf3 : NEG_INF_F;
                A1[r][q] = with_leaf ? A1[r][q] + leaf1 : NEG_INF_F;
            }
        }
    }
    // length 0: nothing; length 1: only the last node (pcfg_viterbi.cu:57-59)
    for (int i = tid; i < 3 * MP; i += NT) col[i] = (i == 1 * MP + mc - 1) ? ob[m - 1] : NEG_INF_F;
    __syncthreads();  // also orders the table fill above before the cells written below
    if (tid == 0 && Lq > 1) Sb[(size_t)(m - 1) * Lq + 1] = ob[m - 1];

    const int len_end = m / 4;  // pcfg_viterbi.cu:67
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int i1 = 1, i2 = 0, i0 = 2;  // column slots of len-1, len-2, len
    for (int len = 2; len < len_end; len++) {
        const float *cur1 = col + i1 * MP, *cur2 = col + i2 * MP;
        float *nxt = col + i0 * MP;
        float sc1[NQ], sc2[NQ];
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            sc1[q] = cur1[j16 + 16 * q];
            sc2[q] = cur2[j16 + 16 * q];
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int a_id = gidx + 64 * r;
            const int row_lo = 64 * r + 4 * wave;  // (as in viterbi_ml1_kernel: passes and chunks without a candidate)
            if (row_lo >= mc) continue;
            float best = NEG_INF_F;
            int sel = -1;
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                if (q >= 4 * r && 16 * q + 15 >= row_lo && 16 * q < mc) {
                    const float c0 = (A0[r][q] + sc1[q]) + ob_a[r];
                    const float c3 = (A3[r][q] + sc2[q]) + ob_a[r];
                    const float c1 = (A1[r][q] + sc2[q]) + ob_a[r];
                    if (c0 > best) {  // false for NaN and for -inf against the initial -inf
                        best = c0;
                        sel = 4 * q;
                    }
                    if (c3 > best) {
                        best = c3;
                        sel = 4 * q + 1;
                    }
                    if (c1 > best) {
                        best = c1;
                        sel = 4 * q + 2;
                    }
                }
            }
            // row maximum first, then the smallest tie key among the lanes that hold it
            const float mine = best;
            best = row16_max_raw(best);
            int key = (sel < 0 || mine != best) ? 0x7fffffff : tie_key3(j16 + 16 * (sel >> 2) - a_id, sel & 3);
            key = min(key, dpp_i<DPP_QUAD_XOR1>(key));
            key = min(key, dpp_i<DPP_QUAD_XOR2>(key));
            key = min(key, dpp_i<DPP_ROW_HALF_MIRROR>(key));
            key = min(key, dpp_i<DPP_ROW_MIRROR>(key));
            if (j16 == 0) {
                nxt[a_id] = best;
                if (best != NEG_INF_F && a_id < mc) {  // pcfg_viterbi.cu:125-131
                    const int a = 4 * a_id + 1;
                    const int option = key & 3, rel = (key >> 2) & 0x3fffff;
                    const unsigned o = (unsigned)(a * Lq + len);  // 32-bit offset from the uniform table bases
                    Sb[o] = best;
                    Lb[o] = option == 0 ? 0 : option == 1 ? a - 3 : a - 1;
                    Rb[o] = 4 * (a_id + rel) + 1;
                    Mb[o] = option ? 1 : 0;
                }
            }
        }
        const int t = i2;
        i2 = i1;
        i1 = i0;
        i0 = t;
        lds_barrier();
    }
}

// ------------------------------------------------------------------------------------------------------------
// Pipelined sweep for the single-call decode of long graphs (same idea as the pipelined inside sweeps): the main chain is
// cut into blocks of 16 parents, one workgroup per block - four compute waves (one 16-lane row per parent, its
// triangular link slabs in registers) and one collector wave.  A parent combines children c >= a only, so the top
// block runs free and every other block follows the one above at the distance of one exchange through memory; the
// score table travels through X [B][Lq][16*NQ] (one entry per length and node, written once by its owner, all ones =
// not arrived, filled by viterbi_pipe_fill_kernel).  The sweep leaves the back-pointer records W and the root's scores;
// viterbi_ml1_kernel<NQ, true> then selects the length and walks the tree (and redoes a sentence whose blocks gave up).
// Values and arg-max decisions are those of viterbi_ml1_kernel: same candidate order inside a lane, same tie key.
// ------------------------------------------------------------------------------------------------------------
constexpr int VP_NT = 16 * 16 + 64;

__global__ __launch_bounds__(256) void viterbi_pipe_fill_kernel(unsigned *X, size_t nx, int *W, size_t nw, float *scores, size_t ns,
                                                               int *flags, int B) {
    const size_t me = (size_t)blockIdx.x * 256 + threadIdx.x, all = (size_t)gridDim.x * 256;
    for (size_t i = me; i < nx; i += all) X[i] = EMPTY32;
    for (size_t i = me; i < nw; i += all) W[i] = 0;
    for (size_t i = me; i < ns; i += all) scores[i] = NEG_INF_F;
    if (me < (size_t)B) flags[me] = 0;
}

template <int NQ>
__global__ __launch_bounds__(VP_NT) void viterbi_ml1_pipe_kernel(const float *__restrict__ ob_lprob, const float *__restrict__ links,
                                                                const int64_t *__restrict__ out_len, int L, int Lq,
                                                                unsigned *__restrict__ X, float *__restrict__ scores,
                                                                int *__restrict__ W, int *__restrict__ flags, int spin_limit) {
    constexpr int MP = 16 * NQ, RQ = (NQ + 3) / 4;  // RQ loads of 64 entries cover a column
    __shared__ float col[3 * MP];
    __shared__ int sm_dead;
    const int b = blockIdx.x / NQ, k = NQ - 1 - blockIdx.x % NQ;  // the leading (highest) block first
    const int tid = threadIdx.x, gidx = (tid >> 4) & 15, j16 = tid & 15, lane = tid & 63;
    const bool collector = tid >= 256;
    const int m = (int)out_len[b];
    if (m < 2 || m > L || (m % 2) != 0) return;  // out of contract: the empty tables stay
    const int mc = m / 2;
    if (16 * k >= mc) return;  // no node of the sentence in this block: nobody waits for it
    const float *ob = ob_lprob + (size_t)b * L;
    const float *lk = links + (size_t)b * L * 2 * L;
    unsigned *Xb = X + (size_t)b * Lq * MP;
    int *Wb = W + (size_t)b * (L / 2) * Lq;

    // slabs: unconditional loads from clamped addresses (all in flight together), masked afterwards
    const int a_id = 16 * k + gidx, a = 2 * min(a_id, mc - 1) + 1;
    float A0[NQ], A1[NQ];
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        A0[q] = A1[q] = NEG_INF_F;
        if (q >= k) {
            const int c = 2 * min(j16 + 16 * q, mc - 1) + 1;
            A0[q] = lk[((size_t)a * 2 + 0) * L + c];
            A1[q] = lk[((size_t)a * 2 + 1) * L + c];
        }
    }
    const float oa = ob[a], ol = ob[a - 1];
    const float ob_a = (a_id < mc) ? oa : NEG_INF_F;
    const float ob_leaf = (a_id < mc && a_id >= 1) ? ol : NEG_INF_F;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
        if (q >= k) {
            const int c_id = j16 + 16 * q;
            const bool ok = a_id < mc && c_id < mc && c_id >= a_id;
            A0[q] = ok ? A0[q] + 0.f : NEG_INF_F;
            A1[q] = (ok && a_id >= 1) ? A1[q] + ob_leaf : NEG_INF_F;
        }
    }
    // length 0: nothing; length 1: only the last node (pcfg_viterbi.cu:57-59)
    for (int i = tid; i < 3 * MP; i += VP_NT) col[i] = (i == 1 * MP + mc - 1) ? ob[m - 1] : NEG_INF_F;
    if (tid == 0) {
        sm_dead = 0;
        if (k == 0 && Lq > 1 && m - 1 == 1) scores[(size_t)b * Lq + 1] = ob[m - 1];
    }
    const int len_end = m / 4;  // pcfg_viterbi.cu:67
    // collector: the entries of the blocks above are requested one step before they are handed on
    unsigned x[RQ];
#pragma unroll
    for (int r = 0; r < RQ; r++)
        x[r] = (collector && len_end > 2) ? entry_load(Xb + (size_t)2 * MP + 16 * (k + 1) + 64 * r + lane) : __float_as_uint(NEG_INF_F);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the slabs have arrived before the sweep starts
    __syncthreads();

    for (int len = 2; len < len_end; len++) {
        const float *cur1 = col + ((len - 1) % 3) * MP, *cur2 = col + ((len - 2) % 3) * MP;
        float *nxt = col + (len % 3) * MP;
        if (collector) {
            // length len of the blocks above; the requests went out for every lane, entries beyond the sentence or the
            // padded row are never written and read as -inf
#pragma unroll
            for (int r = 0; r < RQ; r++)
                if (16 * (k + 1) + 64 * r + lane >= mc) x[r] = __float_as_uint(NEG_INF_F);
            for (int spins = 0;; spins++) {
                bool pending = false;
#pragma unroll
                for (int r = 0; r < RQ; r++) pending |= (x[r] == EMPTY32);
                if (!__any(pending)) break;
                if (spins >= spin_limit || ((spins & 63) == 63 && gave_up(flags + b))) {
                    sm_dead = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
#pragma unroll
                for (int r = 0; r < RQ; r++)
                    if (x[r] == EMPTY32) x[r] = entry_load(Xb + (size_t)len * MP + 16 * (k + 1) + 64 * r + lane);
            }
#pragma unroll
            for (int r = 0; r < RQ; r++) {
                const int i = 16 * (k + 1) + 64 * r + lane;
                if (i < MP) nxt[i] = (x[r] == EMPTY32) ? NEG_INF_F : __uint_as_float(x[r]);
            }
            if (len + 1 < len_end) {
#pragma unroll
                for (int r = 0; r < RQ; r++) x[r] = entry_load(Xb + (size_t)(len + 1) * MP + 16 * (k + 1) + 64 * r + lane);
            }
        } else {
            // the two columns first, all reads in flight together (a read inside each chunk's branch costs the block one
            // LDS round trip per chunk: 106 -> 89 us at 12 blocks), then the chunks that hold children of this block
            float sc1[NQ], sc2[NQ];
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                sc1[q] = cur1[j16 + 16 * q];
                sc2[q] = cur2[j16 + 16 * q];
            }
#pragma unroll
            for (int q = 0; q < NQ; q++) asm volatile("" : "+v"(sc1[q]), "+v"(sc2[q]));  // (keeps the reads up here)
            float best = NEG_INF_F;
            int sel = -1;
            // chunks in groups of four under one branch each (the chunks in front of the block hold -inf in the slabs): a
            // branch per chunk scattered the loop over the kernel's code, and the jumps cost more than the chunks
#pragma unroll
            for (int q4 = 0; q4 < NQ; q4 += 4) {
                if (q4 + 3 >= k) {
#pragma unroll
                    for (int q = q4; q < q4 + 4 && q < NQ; q++) {
                        const float c0 = (A0[q] + sc1[q]) + ob_a;
                        const float c1 = (A1[q] + sc2[q]) + ob_a;
                        if (c0 > best) {  // false for NaN and for -inf against the initial -inf
                            best = c0;
                            sel = 2 * q;
                        }
                        if (c1 > best) {
                            best = c1;
                            sel = 2 * q + 1;
                        }
                    }
                }
            }
            // row maximum first, then the smallest tie key among the lanes that hold it
            const float mine = best;
            best = row16_max_raw(best);
            int key = (sel < 0 || mine != best) ? 0x7fffffff : tie_key(j16 + 16 * (sel >> 1) - a_id, sel & 1);
            key = min(key, dpp_i<DPP_QUAD_XOR1>(key));
            key = min(key, dpp_i<DPP_QUAD_XOR2>(key));
            key = min(key, dpp_i<DPP_ROW_HALF_MIRROR>(key));
            key = min(key, dpp_i<DPP_ROW_MIRROR>(key));
            if (j16 == 0) {
                nxt[a_id] = best;
                if (a_id < mc) {
                    entry_store(Xb + (size_t)len * MP + a_id, best);
                    if (best != NEG_INF_F) {  // pcfg_viterbi.cu:125-131
                        const int jj = key & 1, rel = (key >> 1) & 0x7fffff;
                        Wb[(unsigned)(a_id * Lq + len)] = 1 + ((rel << 1) | jj);
                        if (a_id == 0) scores[(size_t)b * Lq + len] = best;
                    }
                }
            }
        }
        lds_barrier();
        if (sm_dead) {  // uniform: written before the barrier
            if (tid == 0) __hip_atomic_store(flags + b, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
}

// Streaming variant for graphs whose link slabs do not fit in registers (Mc > 256): rows in tiles of 64, link values
// fetched from L2 every step.  LDS: three rotating columns (lengths len, len-1, len-2).
__global__ __launch_bounds__(NT) void viterbi_ml1_stream_kernel(const float *__restrict__ ob_lprob, const float *__restrict__ links,
                                                               const int64_t *__restrict__ out_len, float *__restrict__ S,
                                                               int64_t *__restrict__ Rt, int64_t *__restrict__ Lt,
                                                               int64_t *__restrict__ Mt, int L, int Lq, int MP) {
    extern __shared__ float col[];  // [3][MP]
    const int b = blockIdx.x, tid = threadIdx.x, gidx = tid >> 4, j16 = tid & 15;
    const int m = (int)out_len[b];
    const float *ob = ob_lprob + (size_t)b * L;
    const float *lk = links + (size_t)b * L * 2 * L;
    const size_t tab = (size_t)b * L * Lq;
    float *Sb = S + tab;
    int64_t *Rb = Rt + tab, *Lb = Lt + tab, *Mb = Mt + tab;
    for (size_t i = tid; i < (size_t)L * Lq; i += NT) {
        Sb[i] = NEG_INF_F;
        Rb[i] = 0;
        Lb[i] = 0;
        Mb[i] = 0;
    }
    if (m < 2 || m > L || (m % 2) != 0) return;
    const int mc = m / 2;
    for (int i = tid; i < 3 * MP; i += NT) col[i] = NEG_INF_F;
    __syncthreads();
    if (tid == 0) {
        col[1 * MP + mc - 1] = ob[m - 1];
        if (Lq > 1) Sb[(size_t)(m - 1) * Lq + 1] = ob[m - 1];
    }
    __syncthreads();

    const int ntiles = (mc + 63) / 64;
    const int nq = (mc + 15) / 16;
    const int len_end = m / 4;
    for (int len = 2; len < len_end; len++) {
        const float *cur1 = col + ((len - 1) % 3) * MP, *cur2 = col + ((len - 2) % 3) * MP;
        float *nxt = col + (len % 3) * MP;
        for (int tile = 0; tile < ntiles; tile++) {
            const int a_id = tile * 64 + gidx, a = 2 * a_id + 1;
            const bool row_ok = a_id < mc;
            const float ob_a = row_ok ? ob[a] : NEG_INF_F;
            const float ob_leaf = (row_ok && a_id >= 1) ? ob[a - 1] : NEG_INF_F;
            const float *l0 = lk + ((size_t)a * 2 + 0) * L, *l1 = lk + ((size_t)a * 2 + 1) * L;
            float best = NEG_INF_F;
            int key = 0x7fffffff;
            for (int q = 4 * tile; q < nq; q++) {
                const int c_id = j16 + 16 * q;
                const bool ok = row_ok && c_id < mc && c_id >= a_id;
                const float x0 = ok ? l0[2 * c_id + 1] : NEG_INF_F;
                const float x1 = (ok && a_id >= 1) ? l1[2 * c_id + 1] : NEG_INF_F;
                const float s1 = (c_id < MP) ? cur1[c_id] : NEG_INF_F;
                const float s2 = (c_id < MP) ? cur2[c_id] : NEG_INF_F;
                const float c0 = nan_to_ninf(((x0 + 0.f) + s1) + ob_a);
                const float c1 = nan_to_ninf(((x1 + ob_leaf) + s2) + ob_a);
                const int rel = c_id - a_id;
                if (c0 != NEG_INF_F) take_better(best, key, c0, tie_key(rel, 0));
                if (c1 != NEG_INF_F) take_better(best, key, c1, tie_key(rel, 1));
            }
            row16_argmax_step<DPP_QUAD_XOR1>(best, key);
            row16_argmax_step<DPP_QUAD_XOR2>(best, key);
            row16_argmax_step<DPP_ROW_HALF_MIRROR>(best, key);
            row16_argmax_step<DPP_ROW_MIRROR>(best, key);
            if (j16 == 0 && a_id < MP) {
                nxt[a_id] = best;
                if (best != NEG_INF_F && row_ok) {
                    const int jj = key & 1, rel = (key >> 1) & 0x7fffff;
                    const size_t o = (size_t)a * Lq + len;
                    Sb[o] = best;
                    Lb[o] = jj ? (a - 1) : 0;
                    Rb[o] = 2 * (a_id + rel) + 1;
                    Mb[o] = jj;
                }
            }
        }
        lds_barrier();
    }
}

__global__ void readout_kernel(const int64_t *pred_length, const int64_t *output_length, const int64_t *Lt, const int64_t *Rt,
                               const int64_t *Mt, const int64_t *tokens, const int64_t *mask, int64_t mask_dim, int64_t pad,
                               int64_t *out_tokens, int64_t *out_count, int64_t *scratch, int B, int L, int Lq) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= B) return;
    int64_t *out = out_tokens + (size_t)i * L;
    for (int k = 0; k < L; k++) out[k] = pad;
    const size_t tab = (size_t)i * L * Lq;
    int64_t *stack_node = scratch + (size_t)i * 2 * L, *stack_len = stack_node + L;
    const FullTraces tr{Lt + tab, Rt + tab, Mt + tab, Lq};
    const WalkInputs in{tokens + (size_t)i * L, mask, mask_dim};
    out_count[i] = readout_one(pred_length[i], output_length[i], tr, in, pad, out, stack_node, stack_len, L, Lq);
}

// Length selection on full tables (one wave per sentence): scores[len] = S[b][1][len].
__global__ __launch_bounds__(64) void select_length_kernel(const float *__restrict__ S, const float *__restrict__ penalty,
                                                          int64_t *__restrict__ pred_length, int L, int Lq) {
    const int b = blockIdx.x;
    const int pl = select_length(S + ((size_t)b * L + 1) * Lq, penalty, Lq, threadIdx.x);
    if (threadIdx.x == 0) pred_length[b] = pl;
}

// The emitted tokens as float32 (the general path of the single-call decode; the one-workgroup decode converts its own row).
__global__ __launch_bounds__(256) void tokens_to_float_kernel(const int64_t *__restrict__ tokens, float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = (float)tokens[i];
}

// `lookahead` / `greedy` decode (glat_decomposed_with_link_two_hands_tri_pcfg.py:419-481), one workgroup per sentence:
// every wave takes rows of the sentence's link tensor and finds the first arg max over the flattened (k, c) of
//   (links[a][k][c] + ob[c] * beta) + ob[left(a,k)] * beta     (lookahead, :421-427; left(a,0) = 0, left(a,k) = max(a-k, 0))
//   links[a][k][c]                                              (greedy, ob == null, :432-434)
// in fp32 in this association order; the pointers go to LDS (and to `links_idx`), then one thread walks the tree in
// order (:434-476): left child unless left_tree_mask forbids it, emit the node's token unless it is the pad symbol,
// right child.  Dynamic LDS: pointers [L], stack [L + 4].
__global__ __launch_bounds__(NT) void lookahead_decode_kernel(const float *__restrict__ links, const float *__restrict__ ob_lprob,
                                                             float beta, const int64_t *__restrict__ out_len,
                                                             const int64_t *__restrict__ tokens, const int64_t *__restrict__ mask,
                                                             int64_t mask_dim, int64_t pad, int64_t *__restrict__ links_idx,
                                                             int64_t *__restrict__ out_tokens, int64_t *__restrict__ out_count, int L,
                                                             int K) {
    extern __shared__ int dyn[];
    int *s_idx = dyn;        // [L]
    int *s_stack = dyn + L;  // [L + 4]
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lk = links + (size_t)b * L * K * L;
    const float *ob = ob_lprob ? ob_lprob + (size_t)b * L : nullptr;
    const int row_len = K * L;
    for (int i = tid; i < L; i += NT) out_tokens[(size_t)b * L + i] = pad;
    for (int a = wave; a < L; a += NT / 64) {
        const float *row = lk + (size_t)a * row_len;
        float best = NEG_INF_F;
        int arg = 0x7fffffff;
        for (int i = lane; i < row_len; i += 64) {
            float v = row[i];
            if (ob) {
                const int k = i / L, c = i - k * L;
                const int left = (k == 0) ? 0 : (a - k < 0 ? 0 : a - k);
                const float r = ob[c] * beta, l = ob[left] * beta;
                v = (v + r) + l;
            }
            if (v > best) {  // ascending scan, strict: the first maximum of this lane
                best = v;
                arg = i;
            }
        }
        const float top = wave_max(best);
        const int first = wave_min((best == top && arg != 0x7fffffff) ? arg : 0x7fffffff);
        if (lane == 0) {
            const int r = (first == 0x7fffffff) ? 0 : first;  // a row of -inf: index 0, like torch.max
            s_idx[a] = r;
            if (links_idx) links_idx[(size_t)b * L + a] = r;
        }
    }
    __syncthreads();
    if (tid != 0) return;
    const int64_t length = out_len[b];
    int sp = 0;
    int64_t cnt = 0, now = 1;
    int64_t budget = 4 * (int64_t)L + 8;
    bool bad = false;
    while ((now < length && now != 0) || sp > 0) {
        if (--budget < 0) { bad = true; break; }
        while (now < length && now != 0) {
            if (sp >= L + 4 || now < 0 || now >= L) { bad = true; break; }
            s_stack[sp++] = (int)now;
            const int64_t k = s_idx[now] / L;
            const int64_t left = (k == 0) ? 0 : now - k;
            if (left < 0 || left >= mask_dim || now >= mask_dim) { bad = true; break; }
            if (mask[now * mask_dim + left]) break;
            now = left;
        }
        if (bad) break;
        now = s_stack[--sp];
        const int64_t t = tokens[(size_t)b * L + now];
        if (t != pad) {
            if (cnt < L) out_tokens[(size_t)b * L + cnt] = t;
            else bad = true;
            cnt++;
        }
        now = s_idx[now] % L;
    }
    out_count[b] = bad ? -1 : cnt;
}

}  // namespace
}  // namespace pcfgnat

using namespace pcfgnat;

extern "C" int pcfgnat_lookahead_decode(const float *links, const float *ob_lprob, float beta, const int64_t *output_length,
                                        const int64_t *tokens, const int64_t *left_tree_mask, int64_t mask_dim, int64_t pad_index,
                                        int64_t *links_idx, int64_t *out_tokens, int64_t *out_count, int64_t B, int64_t L,
                                        int64_t ml, void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 2 && ml >= 0 && mask_dim >= 1, "lookahead_decode: bad dimensions");
    PCFGNAT_REQUIRE(L <= 8192 && (ml + 1) * L < (1LL << 30), "lookahead_decode: graph too large");
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(links && output_length && tokens && left_tree_mask && out_tokens && out_count, "lookahead_decode: null pointer");
    const size_t dyn = ((size_t)2 * L + 4) * sizeof(int);
    hipLaunchKernelGGL(lookahead_decode_kernel, dim3((unsigned)B), dim3(NT), dyn, (hipStream_t)stream, links, ob_lprob, beta,
                       output_length, tokens, left_tree_mask, mask_dim, pad_index, links_idx, out_tokens, out_count, (int)L,
                       (int)(ml + 1));
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_pcfg_viterbi(const float *ob_lprob, const float *links, const int64_t *output_length, float *S, int64_t *R,
                                    int64_t *Lt, int64_t *M, int64_t B, int64_t L, int64_t ml, void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 4, "pcfg_viterbi: need B >= 0 and L >= 4 (got B=%lld L=%lld)", (long long)B, (long long)L);
    PCFGNAT_REQUIRE(ml >= 0 && ml <= 63, "pcfg_viterbi: max_left out of range");
    PCFGNAT_REQUIRE(L / 4 > ml, "pcfg_viterbi: L/4 must exceed max_left");
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(ob_lprob && links && output_length && S && R && Lt && M, "pcfg_viterbi: null pointer");
    const int Lq = (int)(L / 4);
    hipStream_t s = (hipStream_t)stream;
    if (ml == 3 && viterbi_ml3_supported(L)) {
        // the sentences without a rule of a composite local tree in one launch, the others by the general kernel behind
        const int Mc3 = (int)((L - 2) / 4 + 1);
#define PCFGNAT_VITERBI3_CASE(nq)                                                                                             \
    else if (Mc3 <= 16 * (nq))                                                                                               \
        hipLaunchKernelGGL((viterbi_ml3_kernel<nq>), dim3((unsigned)B), dim3(NT), 0, s, ob_lprob, links, output_length, S, R, Lt, M, \
                           (int)L, Lq)
        if (false) {
        }
        PCFGNAT_VITERBI3_CASE(2);
        PCFGNAT_VITERBI3_CASE(4);
        PCFGNAT_VITERBI3_CASE(6);
        PCFGNAT_VITERBI3_CASE(8);
#undef PCFGNAT_VITERBI3_CASE
        PCFGNAT_HIP_CHECK(hipGetLastError());
        return generic_viterbi(ob_lprob, links, output_length, S, R, Lt, M, B, L, ml, stream, 1);
    }
    if (ml != 1) return generic_viterbi(ob_lprob, links, output_length, S, R, Lt, M, B, L, ml, stream);
    const int Mc = (int)((L - 2) / 2 + 1);
#define PCFGNAT_VITERBI_CASE(nq)                                                                                              \
    else if (Mc <= 16 * (nq))                                                                                                \
        hipLaunchKernelGGL((viterbi_ml1_kernel<nq, false>), dim3((unsigned)B), dim3(NT), 0, s, ob_lprob, links, output_length, S, R, Lt, \
                           M, (int)L, Lq, DecodeArgs{})
    if (false) {
    }
    PCFGNAT_VITERBI_CASE(2);
    PCFGNAT_VITERBI_CASE(4);
    PCFGNAT_VITERBI_CASE(6);
    PCFGNAT_VITERBI_CASE(8);
    PCFGNAT_VITERBI_CASE(10);
    PCFGNAT_VITERBI_CASE(12);
    PCFGNAT_VITERBI_CASE(14);
    PCFGNAT_VITERBI_CASE(16);
#undef PCFGNAT_VITERBI_CASE
    else {
        PCFGNAT_REQUIRE(L <= 4096, "pcfg_viterbi: graph size L=%lld exceeds 4096 nodes", (long long)L);
        const int MP = ((Mc + 63) / 64) * 64;
        hipLaunchKernelGGL(viterbi_ml1_stream_kernel, dim3((unsigned)B), dim3(NT), (size_t)3 * MP * sizeof(float), s, ob_lprob, links,
                           output_length, S, R, Lt, M, (int)L, Lq, MP);
    }
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

namespace {
// the single-launch decode applies to max_left = 1 graphs whose slabs fit in registers
bool decode_is_fused(int64_t L, int64_t ml) { return ml == 1 && (L - 2) / 2 + 1 <= 256; }
// 16-node chunks of the main chain, rounded to the kernels that exist (2, 4, .., 16)
int decode_chunks(int64_t L) { return 2 * (int)(((L - 2) / 2 + 1 + 31) / 32); }
// The pipelined sweep pays from about 200 graph nodes on while every block gets a compute unit of its own, from about
// 260 nodes otherwise (measured: batch 1, 240 nodes 132 -> 123 us per call, 400 nodes 322 -> 192 us; batch 64, 200 nodes
// 125 -> 134 us, 400 nodes 338 -> 231 us); below that one workgroup is through before a pipeline has filled.
bool decode_pipelined(int NQ, int64_t B) {
    if (B * NQ > pipeline_max_workgroups()) return false;
    return NQ >= 10 || (NQ >= 8 && B * NQ <= 256);
}

template <int NQ>
int launch_decode(const float *ob_lprob, const float *links, const int64_t *output_length, DecodeArgs dec, void *workspace, int64_t B,
                  int64_t L, hipStream_t s) {
    const int Lq = (int)(L / 4);
    const size_t dyn = (size_t)L * sizeof(int64_t) + (size_t)Lq * sizeof(int) + (size_t)L;
    const size_t nw = (size_t)B * (size_t)(L / 2) * Lq, nx = (size_t)B * Lq * 16 * NQ, ns = (size_t)B * Lq;
    if (decode_pipelined(NQ, B)) {
        int *W = (int *)workspace;
        unsigned *X = (unsigned *)(W + nw);
        float *scores = (float *)(X + nx);
        int *flags = (int *)(scores + ns);
        const size_t total = nw + nx + ns;
        const unsigned fill_blocks = (unsigned)((total / 4 + 255) / 256 < 1024 ? (total / 4 + 255) / 256 : 1024);
        hipLaunchKernelGGL(viterbi_pipe_fill_kernel, dim3(fill_blocks ? fill_blocks : 1), dim3(256), 0, s, X, nx, W, nw, scores, ns, flags,
                           (int)B);
        PCFGNAT_HIP_CHECK(hipGetLastError());
        hipLaunchKernelGGL(viterbi_ml1_pipe_kernel<NQ>, dim3((unsigned)(B * NQ)), dim3(VP_NT), 0, s, ob_lprob, links, output_length, (int)L,
                           Lq, X, scores, W, flags, pipeline_spin_limit());
        PCFGNAT_HIP_CHECK(hipGetLastError());
        dec.pipe_flags = flags;
        dec.pipe_scores = scores;
    }
    hipLaunchKernelGGL((viterbi_ml1_kernel<NQ, true>), dim3((unsigned)B), dim3(NT), dyn, s, ob_lprob, links, output_length, nullptr, nullptr,
                       nullptr, nullptr, (int)L, Lq, dec);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}
}  // namespace

extern "C" size_t pcfgnat_viterbi_decode_workspace_bytes(int64_t B, int64_t L, int64_t ml) {
    if (B <= 0 || L < 4) return 0;
    const size_t Lq = (size_t)(L / 4);
    // back-pointer records [B][L/2][Lq], then (pipelined sweep) the score exchange [B][Lq][16*chunks], root scores [B][Lq], flags [B]
    if (decode_is_fused(L, ml))
        return ((size_t)B * (size_t)(L / 2) * Lq + (size_t)B * Lq * 16 * decode_chunks(L) + (size_t)B * Lq + (size_t)B) * sizeof(int);
    // full tables S (float) + R, L, M (int64), then the walk stacks [B][2L] int64
    return (size_t)B * L * Lq * (sizeof(float) + 3 * sizeof(int64_t)) + (size_t)B * 2 * L * sizeof(int64_t);
}

extern "C" int pcfgnat_viterbi_decode(const float *ob_lprob, const float *links, const int64_t *output_length, const int64_t *tokens,
                                      const int64_t *left_tree_mask, int64_t mask_dim, int64_t pad_index, const float *length_penalty,
                                      void *workspace, int64_t *out_tokens, float *out_tokens_f32, int64_t *out_count,
                                      int64_t *pred_length, int64_t B, int64_t L, int64_t ml, void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 4, "viterbi_decode: need B >= 0 and L >= 4 (got B=%lld L=%lld)", (long long)B, (long long)L);
    PCFGNAT_REQUIRE(ml >= 0 && ml <= 63 && L / 4 > ml, "viterbi_decode: max_left out of range for this graph size");
    PCFGNAT_REQUIRE(mask_dim >= 1, "viterbi_decode: bad mask dimension");
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(ob_lprob && links && output_length && tokens && left_tree_mask && length_penalty && workspace && out_tokens &&
                        out_count && pred_length,
                    "viterbi_decode: null pointer");
    PCFGNAT_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7) == 0, "viterbi_decode: workspace must be 8-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int Lq = (int)(L / 4);
    if (decode_is_fused(L, ml)) {
        DecodeArgs dec{tokens,      left_tree_mask, length_penalty, (int *)workspace, out_tokens, out_count,
                       pred_length, out_tokens_f32, mask_dim,       pad_index,        nullptr,    nullptr};
        switch (decode_chunks(L)) {
            case 2: return launch_decode<2>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            case 4: return launch_decode<4>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            case 6: return launch_decode<6>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            case 8: return launch_decode<8>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            case 10: return launch_decode<10>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            case 12: return launch_decode<12>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            case 14: return launch_decode<14>(ob_lprob, links, output_length, dec, workspace, B, L, s);
            default: return launch_decode<16>(ob_lprob, links, output_length, dec, workspace, B, L, s);
        }
    }
    // general path: full tables in the workspace, then selection and walk as separate launches
    const size_t cells = (size_t)B * L * Lq;
    int64_t *Rw = (int64_t *)workspace, *Lw = Rw + cells, *Mw = Lw + cells, *stacks = Mw + cells;
    float *Sw = (float *)(stacks + (size_t)B * 2 * L);
    int rc = pcfgnat_pcfg_viterbi(ob_lprob, links, output_length, Sw, Rw, Lw, Mw, B, L, ml, stream);
    if (rc != PCFGNAT_OK) return rc;
    hipLaunchKernelGGL(select_length_kernel, dim3((unsigned)B), dim3(64), 0, s, Sw, length_penalty, pred_length, (int)L, Lq);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    rc = pcfgnat_viterbi_decoding(pred_length, output_length, Lw, Rw, Mw, tokens, left_tree_mask, mask_dim, pad_index, out_tokens,
                                  out_count, stacks, B, L, Lq, stream);
    if (rc != PCFGNAT_OK || out_tokens_f32 == nullptr) return rc;
    const size_t cells_out = (size_t)B * L;
    hipLaunchKernelGGL(tokens_to_float_kernel, dim3((unsigned)((cells_out + 255) / 256)), dim3(256), 0, s, out_tokens, out_tokens_f32,
                       cells_out);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_viterbi_decoding(const int64_t *pred_length, const int64_t *output_length, const int64_t *Lt, const int64_t *R,
                                        const int64_t *M, const int64_t *tokens, const int64_t *left_tree_mask, int64_t mask_dim,
                                        int64_t pad_index, int64_t *out_tokens, int64_t *out_count, int64_t *scratch, int64_t B,
                                        int64_t L, int64_t Lq, void *stream) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 1 && Lq >= 1 && mask_dim >= 1, "viterbi_decoding: bad dimensions");
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(pred_length && output_length && Lt && R && M && tokens && left_tree_mask && out_tokens && out_count && scratch,
                    "viterbi_decoding: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const int threads = 64;
    hipLaunchKernelGGL(readout_kernel, dim3((unsigned)((B + threads - 1) / threads)), dim3(threads), 0, s, pred_length, output_length, Lt,
                       R, M, tokens, left_tree_mask, mask_dim, pad_index, out_tokens, out_count, scratch, (int)B, (int)L, (int)Lq);
    PCFGNAT_HIP_CHECK(hipGetLastError());
    return PCFGNAT_OK;
}

extern "C" int pcfgnat_viterbi_decoding_host(const int64_t *pred_length, const int64_t *output_length, const int64_t *Lt,
                                             const int64_t *R, const int64_t *M, const int64_t *tokens, const int64_t *left_tree_mask,
                                             int64_t mask_dim, int64_t pad_index, int64_t *out_tokens, int64_t *out_count, int64_t B,
                                             int64_t L, int64_t Lq) {
    PCFGNAT_REQUIRE(B >= 0 && L >= 1 && Lq >= 1 && mask_dim >= 1, "viterbi_decoding: bad dimensions");
    if (B == 0) return PCFGNAT_OK;
    PCFGNAT_REQUIRE(pred_length && output_length && Lt && R && M && tokens && left_tree_mask && out_tokens && out_count,
                    "viterbi_decoding: null pointer");
    int64_t *stack = (int64_t *)malloc(sizeof(int64_t) * 2 * (size_t)L);
    if (!stack) return fail(PCFGNAT_EINVAL, "viterbi_decoding: out of host memory");
    for (int64_t i = 0; i < B; i++) {
        int64_t *out = out_tokens + (size_t)i * L;
        for (int64_t k = 0; k < L; k++) out[k] = pad_index;
        const size_t tab = (size_t)i * L * Lq;
        const FullTraces tr{Lt + tab, R + tab, M + tab, (int)Lq};
        const WalkInputs in{tokens + (size_t)i * L, left_tree_mask, mask_dim};
        out_count[i] = readout_one(pred_length[i], output_length[i], tr, in, pad_index, out, stack, stack + L, (int)L, (int)Lq);
    }
    free(stack);
    return PCFGNAT_OK;
}

bool pcfgnat::viterbi_ml3_supported(int64_t L) { return ml3_tuned_on() && L >= 6 && (L - 2) / 4 + 1 <= 128; }

extern "C" int pcfgnat_max_left3_viterbi_counts(unsigned long long *served, unsigned long long *left_to_plain, int reset) {
    unsigned long long h[2] = {0, 0};
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(h, HIP_SYMBOL(pcfgnat::g_viterbi_ml3_counts), sizeof(h)));
    if (served) *served = h[0];
    if (left_to_plain) *left_to_plain = h[1];
    if (reset) {
        const unsigned long long z[2] = {0, 0};
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(pcfgnat::g_viterbi_ml3_counts), z, sizeof(z)));
    }
    return PCFGNAT_OK;
}

int pcfgnat::viterbi_redo_count(unsigned long long *count, int reset) {
    PCFGNAT_HIP_CHECK(hipMemcpyFromSymbol(count, HIP_SYMBOL(g_viterbi_redone), sizeof(*count)));
    if (reset) {
        const unsigned long long zero = 0;
        PCFGNAT_HIP_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_viterbi_redone), &zero, sizeof(zero)));
    }
    return PCFGNAT_OK;
}
