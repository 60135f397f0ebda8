"""Seeded synthetic inputs shaped like the PCFG-NAT training / decoding batches.

The reference ships no data; these generators reproduce the *support* of what its model emits:

* ``links[b, a, k, c]`` is a joint log-softmax over ``(k, c)`` of ``ab[a, idx(a, k)] + ac[a, c]`` restricted to the
  support tree of ``models/lemon_tree.py:41-119`` as used by ``extract_links``
  (``models/glat_decomposed_with_link_two_hands_tri_pcfg.py:168-199``): only main-chain parents ``a`` (ids
  ``1, ml+2, 2ml+3, ...``) with ``a < m-1`` have finite rows; right children are main-chain nodes ``a < c < m``;
  left option ``k = 0`` is the null node, ``k >= 1`` is node ``a-k`` of the parent's own left subtree; for the root
  ``a = 1`` the gather index clamps to node 0 (``_max_left_index``, same file :213-218), which yields finite duplicates
  of the null option that no kernel ever reads.
* targets carry bos(0) first, eos(2) last, pad(1) beyond the sentence, like fairseq dictionaries.

Everything is drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in a fixed order so that every machine
sees identical bits.
"""
import math

import torch

BOS, PAD, EOS = 0, 1, 2


def support_masks(L, ml):
    """Closed form of the three masks of ``BinaryTreeNode.get_mask`` (lemon_tree.py:92-119) for a graph of ``L`` nodes:
    returns (left_tree_mask [L,L], right_tree_mask [L,L], main_chain [L]) with 1 = forbidden in the two masks, as the
    model passes them to ``viterbi_decoding``.  Only full groups are generated (``(L-2) % (ml+1) == 0``)."""
    g = ml + 1
    left = torch.ones(L, L, dtype=torch.int64)
    right = torch.ones(L, L, dtype=torch.int64)
    main = torch.zeros(L, dtype=torch.bool)
    n_main = (L - 2) // g + 1
    mains = [1 + i * g for i in range(n_main) if 1 + i * g < L]
    for a in mains:
        main[a] = True
    # root: left subtree is node 0 only.
    left[1, 0] = 0
    for a in mains:
        # everything to the right of a main-chain node hangs under its right child
        right[a, a + 1:] = 0
        if a > 1:
            left[a, a - ml:a] = 0
            # inside the complete binary left subtree (in-order ids a-ml .. a-1)
            def fill(lo, hi):  # subtree occupying ids [lo, hi]
                if lo > hi:
                    return
                root = (lo + hi) // 2
                if lo <= root - 1:
                    left[root, lo:root] = 0
                if root + 1 <= hi:
                    right[root, root + 1:hi + 1] = 0
                fill(lo, root - 1)
                fill(root + 1, hi)
            fill(a - ml, a - 1)
    left[1:, 0] = 0
    return left, right, main


def make_links(B, L, out_len, ml=1, generator=None, dtype=torch.float32):
    """Masked, jointly normalised link log-probabilities ``[B, L, ml+1, L]`` (see module docstring)."""
    g = ml + 1
    ab = torch.randn(B, L, L, generator=generator, dtype=torch.float32)
    ac = torch.randn(B, L, L, generator=generator, dtype=torch.float32)
    a_ids = torch.arange(L)
    idx = torch.zeros(L, ml + 1, dtype=torch.int64)
    for k in range(1, ml + 1):
        idx[:, k] = (a_ids - k).clamp(min=0)
    left_term = torch.gather(ab, 2, idx.view(1, L, ml + 1).expand(B, -1, -1))  # [B,L,ml+1]
    raw = left_term.unsqueeze(-1) + ac.unsqueeze(2)  # [B,L,ml+1,L]
    is_main = (a_ids % g == 1) if g > 1 else (a_ids >= 1)
    m = out_len.view(B, 1, 1, 1)
    a4 = a_ids.view(1, L, 1, 1)
    c4 = a_ids.view(1, 1, 1, L)
    k4 = torch.arange(ml + 1).view(1, 1, ml + 1, 1)
    valid = is_main.view(1, L, 1, 1) & (a4 < m - 1) & is_main.view(1, 1, 1, L) & (c4 > a4) & (c4 < m)
    left_ok = (k4 == 0) | (a4 - k4 >= 1) | (a4 == 1)
    valid = valid & left_ok
    raw = raw.masked_fill(~valid, float("-inf"))
    flat = raw.view(B, L, (ml + 1) * L)
    nouse = ~valid.view(B, L, -1).any(-1, keepdim=True)
    flat = torch.log_softmax(flat.masked_fill(nouse, 0.0), dim=-1).masked_fill(nouse, float("-inf"))
    flat = flat.masked_fill(~valid.view(B, L, -1), float("-inf"))
    return flat.view(B, L, ml + 1, L).to(dtype).contiguous()


def make_targets(B, T, tgt_len, V, generator=None):
    tgt = torch.randint(4, V, (B, T), generator=generator, dtype=torch.int64)
    pos = torch.arange(T).view(1, T)
    tgt = tgt.masked_fill(pos >= tgt_len.view(B, 1), PAD)
    tgt[:, 0] = BOS
    tgt.scatter_(1, (tgt_len - 1).view(B, 1), EOS)
    return tgt


def training_batch(B, L, T, V, out_len, tgt_len, seed, ml=1, logit_scale=1.0, logit_dtype=torch.float32):
    """A training-shaped batch: dict with logits [B,L,V], links [B,L,ml+1,L], targets [B,T], output_length,
    target_length.  Draw order: links (ab, ac), targets, logits."""
    gen = torch.Generator().manual_seed(seed)
    out_len = torch.as_tensor(out_len, dtype=torch.int64)
    tgt_len = torch.as_tensor(tgt_len, dtype=torch.int64)
    links = make_links(B, L, out_len, ml, gen)
    targets = make_targets(B, T, tgt_len, V, gen)
    logits = torch.randn(B, L, V, generator=gen, dtype=torch.float32)
    if logit_scale != 1.0:
        logits.mul_(logit_scale)
    logits = logits.to(logit_dtype)
    return {"logits": logits, "links": links, "targets": targets, "output_length": out_len, "target_length": tgt_len,
            "ml": ml}


def config1():
    """Tiny plumbing case: B=2, src 8 -> L=32 nodes, T=10, V=512, fp32 logits ~N(0,1), seed 0."""
    B, L, T, V = 2, 32, 10, 512
    return training_batch(B, L, T, V, [32, 32], [10, 10], seed=0)


def _wmt_lengths(B, gen, src_lo, src_hi, T):
    src = torch.randint(src_lo, src_hi + 1, (B,), generator=gen)
    src[0] = src_hi
    jitter = torch.randint(-2, 3, (B,), generator=gen)
    n = (torch.round(1.1 * src.double()).long() + jitter).clamp(min=2, max=T)
    n[0] = T
    return 4 * src, n


def config2(B=40, L=128, T=32, V=40000, seed=1, logit_dtype=torch.float16):
    """WMT14 En-De shaped training batch: src ~U{10..32} upsampled x4, padded to L=128, T=32, V=40000, fp16 logits
    ~N(0,2)."""
    gen = torch.Generator().manual_seed(seed + 1000)
    m, n = _wmt_lengths(B, gen, 10, L // 4, T)
    return training_batch(B, L, T, V, m, n, seed=seed, logit_scale=2.0, logit_dtype=logit_dtype)


def config3(B=8, L=512, T=140, V=40000, seed=2, logit_dtype=torch.float16):
    """Long-sentence stress: src 128 -> L=512, T=140."""
    return training_batch(B, L, T, V, [L] * B, [T] * B, seed=seed, logit_scale=2.0, logit_dtype=logit_dtype)


def decode_batch(src_lens, seed, V=40000, ml=1, logit_scale=3.0, logit_dtype=torch.float16, L=None):
    """Decoding-shaped batch for the given source lengths: graph size m = 4*src, padded to L = max m (or the given L).
    Returns dict with logits [B,L,V], links, output_length."""
    gen = torch.Generator().manual_seed(seed)
    src = torch.as_tensor(src_lens, dtype=torch.int64)
    m = 4 * src
    B = src.numel()
    if L is None:
        L = int(m.max())
    links = make_links(B, L, m, ml, gen)
    logits = (torch.randn(B, L, V, generator=gen, dtype=torch.float32) * logit_scale).to(logit_dtype)
    return {"logits": logits, "links": links, "output_length": m, "ml": ml}


def config4_lengths(n_sent=1000, seed=3):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(5, 101, (n_sent,), generator=gen)


def ob_and_tokens(logits):
    """Per-node best token and its log-probability, computed once by the harness and fed to every path
    (models/glat_decomposed_with_link_two_hands_tri_pcfg.py:414-415)."""
    lp = torch.log_softmax(logits.float(), dim=-1)
    ob, tok = lp.max(dim=-1)
    return ob.contiguous(), tok.contiguous()


def links_bytes(B, L, ml):
    return B * L * (ml + 1) * L * 4


def lsg_fwd_bytes(B, L, V, T, itemsize, require_grad=True, live_rows=None):
    """Algorithmic HBM bytes of one logsoftmax_gather forward: logits read once, gathered fp32 written, un-expanded int64
    targets read; plus the softmax written in place (reference split, ``require_grad``) or one fp32 log-sum-exp per row.
    ``live_rows``: rows whose logits are read at all (the criterion step skips the pad nodes behind each graph)."""
    rows = B * L if live_rows is None else live_rows
    return (2 if require_grad else 1) * rows * V * itemsize + B * L * T * 4 + B * T * 8 + (0 if require_grad else B * L * 4)


def lsg_bwd_bytes(B, L, V, T, itemsize, live_rows=None, pads_zeroed_elsewhere=False):
    """Algorithmic HBM bytes of the in-place backward: probabilities (or logits) read, gradients written, grad_output read.
    ``live_rows``: rows that are read; the others (pad nodes in the criterion step) are only written - or not touched at
    all when another launch has zeroed them (``pads_zeroed_elsewhere``: graphs of up to 128 nodes, where the launch that
    holds the inside and outside sweeps does it beside them)."""
    rows = B * L if live_rows is None else live_rows
    written = rows if pads_zeroed_elsewhere else B * L
    return (rows + written) * V * itemsize + rows * T * 4


def _selfcheck():  # pragma: no cover
    b = config1()
    assert math.isfinite(float(b["links"][0, 1, 0, 3]))


if __name__ == "__main__":  # pragma: no cover
    _selfcheck()
