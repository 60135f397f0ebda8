"""Test infrastructure: a plain-torch restatement of the link scorer of PCFG-NAT, written from the formulas of
fs_plugins/models/glat_decomposed_with_link_two_hands_tri_pcfg.py:140-201 (`extract_links`), starting after its four
linear projections.  Used only by tests and by bench.py's comparison leg; never by the product path.

For parent a, left option k (k = 0: the null node 0, k >= 1: node a-k) and right child c, per attention head h

    z[a,k,c,h] = ( q[a,h].kl[left(a,k),h] + kl[src(a,k),h].kr[c,h] + q[a,h].kr[c,h] ) / sqrt(F)

with left(a,0) = 0, left(a,k) = max(a-k, 0) (:187, the `_max_left_index` table of :214-218) and src(a,0) = 0,
src(a,k) = (a-1) + (k-1) taken cyclically (:189-193: unfold over windows of max_left rows, rolled by one row).  The
reference's concatenation at :193 only type-checks for max_left = 1, the value every shipped script uses; src(a,1) is
then a-1 (and L-1 for a = 0).  Entries whose left option or right child is masked are -inf (:183-184), rows without any
allowed left option or right child are computed unmasked and overwritten with -inf at the end (:176-181, :199).

    links[a,k,c] = logsumexp_h( log_softmax_h(gate[a,:])[h] + log_softmax_{(k,c)}( z[a,:,:,h] )[k,c] )      (:168, 197-198)
"""
import math

import torch


def link_masks(prev_output_tokens, pad, left_tree_mask, right_tree_mask, main_chain):
    """(:171-181) returns (left forbidden [B,L,L], right forbidden [B,L,L], row unusable [B,L,1]); True = forbidden."""
    is_pad = prev_output_tokens.eq(pad).unsqueeze(1)
    left = torch.logical_or(is_pad, left_tree_mask.bool().unsqueeze(0))
    right = torch.logical_or(is_pad, right_tree_mask.bool().unsqueeze(0))
    right = ~(~right & main_chain.bool().view(1, 1, -1))
    left_nouse = (~left).sum(dim=2, keepdim=True) == 0
    right_nouse = (~right).sum(dim=2, keepdim=True) == 0
    left = left.masked_fill(left_nouse, False)
    right = right.masked_fill(right_nouse, False)
    return left, right, torch.logical_or(left_nouse, right_nouse)


def safe_logsumexp(x, dim):
    """log-sum-exp whose all -inf slices give -inf with a zero (not NaN) gradient, as the model's own helper does (:41-46):
    the maximum is replaced by 0 where it is -inf before it is subtracted."""
    m = x.max(dim=dim)[0]
    dead = m == float("-inf")
    shift = m.masked_fill(dead, 0)
    s = (x - shift.unsqueeze(dim)).exp().sum(dim=dim)
    return s.masked_fill(dead, 1).log() + shift.masked_fill(dead, float("-inf"))


def extract_links(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad, left_tree_mask,
                  right_tree_mask, main_chain, max_left=1):
    """query/key chunks [B,L,H,F], gate_logits [B,L,H] -> links [B,L,max_left+1,L] float32 (differentiable)."""
    if max_left != 1:
        raise ValueError("the reference's construction is only defined for max_left = 1")
    B, L, H, F = query_chunks.shape
    q, kl, kr = query_chunks.float(), key_chunks_left.float(), key_chunks_right.float()
    scale = F ** 0.5
    log_gates = torch.log_softmax(gate_logits, dim=-1, dtype=torch.float)
    ab = torch.einsum("bicf,bjcf->bijc", q, kl) / scale
    ac = torch.einsum("bicf,bjcf->bijc", q, kr) / scale
    bc_folded = torch.einsum("bicf,bjcf->bijc", kl, kr) / scale
    left, right, nouse = link_masks(prev_output_tokens, pad, left_tree_mask, right_tree_mask, main_chain)
    ninf = float("-inf")
    ab = ab.masked_fill(left.view(B, L, L, 1), ninf)
    ac = ac.masked_fill(right.view(B, L, L, 1), ninf)
    index = torch.arange(L, device=q.device).view(1, L, 1).repeat(1, 1, max_left + 1)
    index[:, :, 0] = 0
    for k in range(1, max_left + 1):
        index[:, :, k] = (index[:, :, k] - k).clamp(min=0)
    ab = torch.gather(ab, 2, index.view(1, L, max_left + 1, 1).expand(B, -1, -1, H))
    bc = bc_folded.unfold(1, max_left, 1)
    bc = torch.roll(bc, 1, 1).permute(0, 1, 4, 2, 3)
    bc = torch.cat((bc_folded[:, 0].view(B, 1, 1, L, H).expand(-1, L, -1, -1, -1), bc), 2)
    abc = ab.unsqueeze(3) + bc + ac.unsqueeze(2)
    abc = torch.log_softmax(abc.reshape(B, L, (max_left + 1) * L, H), dim=2)
    links = safe_logsumexp(abc + log_gates.unsqueeze(2), dim=-1).view(B, L, max_left + 1, L)
    return links.masked_fill(nouse.view(B, L, 1, 1), ninf)


def extract_links_loops(q, kl, kr, gate_logits, prev_output_tokens, pad, left_tree_mask, right_tree_mask, main_chain):
    """The same quantity from explicit loops over (b, a, k, c, h) in float64 with its own index arithmetic (max_left = 1):
    the independent check of the tensor expression above.  Small inputs only."""
    B, L, H, F = q.shape
    q, kl, kr = q.double(), kl.double(), kr.double()
    lg = torch.log_softmax(gate_logits.double(), -1)
    out = torch.full((B, L, 2, L), -math.inf, dtype=torch.float64)
    for b in range(B):
        pad_b = [bool(prev_output_tokens[b, j] == pad) for j in range(L)]
        for a in range(L):
            left_ok = [not (pad_b[j] or bool(left_tree_mask[a, j])) for j in range(L)]
            right_ok = [not (pad_b[j] or bool(right_tree_mask[a, j])) and bool(main_chain[j]) for j in range(L)]
            if not any(left_ok) or not any(right_ok):
                continue
            per_head = []
            for h in range(H):
                z = torch.full((2, L), -math.inf, dtype=torch.float64)
                for k in range(2):
                    lft = 0 if k == 0 else max(a - 1, 0)
                    src = 0 if k == 0 else (a - 1) % L
                    if not left_ok[lft]:
                        continue
                    for c in range(L):
                        if right_ok[c]:
                            z[k, c] = (q[b, a, h] @ kl[b, lft, h] + kl[b, src, h] @ kr[b, c, h] + q[b, a, h] @ kr[b, c, h]) / math.sqrt(F)
                per_head.append(lg[b, a, h] + z - torch.logsumexp(z.view(-1), 0))
            out[b, a] = torch.logsumexp(torch.stack(per_head, -1), -1)
    return out
