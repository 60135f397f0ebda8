"""The glue the reference wraps around the ops, restated without fairseq so that the path can be driven end to end:

* ``compute_pcfg_loss``   <- ``NATPCFGoss._compute_pfcg_loss``   (fs_plugins/criterions/nat_pcfg_loss.py:98-145)
* ``glat_alignment``      <- ``glat_function``                    (fs_plugins/criterions/nat_pcfg_loss.py:193-269)
* ``viterbi_decode``      <- the ``viterbi`` branch of ``forward_decoder``
                             (fs_plugins/models/glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416, 483-502)

Each function takes the ops as a namespace argument (``ops``), by default this package's HIP-backed ones, so that tests
can run the very same glue over the CPU oracle.
"""
import torch

from . import custom_ops as _default_ops
from .synth import PAD


def eos_masked(match_all, output_length, target_length):
    """Only the last graph node may emit the last target token (nat_pcfg_loss.py:111-115)."""
    batch_size = match_all.shape[0]
    eos_mask = torch.zeros_like(match_all, dtype=torch.bool)
    rows = torch.arange(batch_size, device=match_all.device)
    eos_mask[rows, :, target_length - 1] = True
    eos_mask[rows, output_length - 1, target_length - 1] = False
    return match_all.masked_fill(eos_mask, float("-inf"))


def compute_pcfg_loss(outputs, output_masks, targets, target_masks, links, ops=_default_ops, matchmask=None, keep_word_mask=None,
                      no_force_emit=False):
    """loss = -(log-likelihood / target_length).mean() with invalid sentences zeroed (nat_pcfg_loss.py:98-145).
    ``outputs`` [B,L,V] is consumed in place (it must not be used afterwards and holds the gradient after backward).  ``matchmask`` [B,T,L] / ``keep_word_mask`` [B,L] (from the glancing step): unless ``no_force_emit``, a
    revealed graph node may only emit the target position it is aligned to, through a detached value (:116-121).
    Returns a dict with ``loss``, ``ll`` (per sentence), ``invalid_nsentences``."""
    prelen = outputs.shape[1]
    output_length = output_masks.sum(dim=-1)
    target_length = target_masks.sum(dim=-1)
    outputs, match_all = ops.dag_logsoftmax_gather_inplace(outputs, targets.unsqueeze(1).expand(-1, prelen, -1))
    match_all_eos_masked = eos_masked(match_all, output_length, target_length)
    if matchmask is not None and not no_force_emit:
        glat_prev_mask = keep_word_mask.unsqueeze(-1)
        mm = matchmask.transpose(1, 2)
        match_all_eos_masked = (match_all_eos_masked.masked_fill(glat_prev_mask, 0) +
                                match_all_eos_masked.masked_fill(~mm, float("-inf")).masked_fill(~glat_prev_mask, 0).detach())
    loss_result = ops.cuda_pcfg_loss(match_all_eos_masked, links, output_length, target_length)
    invalid_masks = loss_result.isinf().logical_or(loss_result.isnan())
    loss_result = loss_result.masked_fill(invalid_masks, 0)
    loss = -(loss_result / target_length).mean()
    return {"loss": loss, "ll": loss_result, "invalid_nsentences": invalid_masks.sum().detach(),
            "match_all": match_all_eos_masked}


def glat_alignment(word_ins_out, tgt_tokens, prev_output_tokens, links, context_p, pad=PAD, ops=_default_ops,
                   generator=None, noise_device=None, single_call=False, glance_strategy="number-random"):
    """GLAT glancing (nat_pcfg_loss.py:193-269): best-tree alignment of target tokens to graph nodes, then a random
    subset of the aligned nodes is revealed, chosen by the criterion's ``glance_strategy``: ``"number-random"`` (every
    shipped script; :235-242), ``"cmlm"`` (:244-251) or ``None`` (:231-233).  RNG order as in the reference: ``randn``
    (not for ``None``), ``rand`` over the batch (``cmlm`` only), ``rand`` over the nodes.  The reference draws on the
    tokens' device; ``noise_device`` (e.g. "cpu") draws elsewhere and moves the numbers, which makes a run reproducible
    across devices.  ``single_call``: the same pass as one native call (``ops.pcfg_glat_step``)."""
    if glance_strategy not in ("number-random", "cmlm", None):
        raise RuntimeError("glat_alignment: unknown glance strategy %r" % (glance_strategy,))
    if single_call:
        return ops.pcfg_glat_step(word_ins_out, tgt_tokens, prev_output_tokens, links, context_p, pad, generator=generator,
                                  noise_device=noise_device, glance_strategy=glance_strategy)
    batch_size, prelen = links.shape[0], links.shape[1]
    tarlen = tgt_tokens.shape[1]
    target_length = (~tgt_tokens.eq(pad)).sum(1)
    output_length = prev_output_tokens.ne(pad).sum(1)
    pred_tokens = word_ins_out.argmax(-1)
    word_ins_out, match = ops.dag_logsoftmax_gather_inplace(word_ins_out, tgt_tokens.unsqueeze(1).expand(-1, prelen, -1))
    match_all_eos_masked = eos_masked(match, output_length, target_length)
    path, max_tree_lprob = ops.cuda_pcfg_best_tree(match_all_eos_masked, links, output_length, target_length)
    invalid_masks = max_tree_lprob.isinf().logical_or(max_tree_lprob.isnan())
    max_tree_lprob = max_tree_lprob.masked_fill(invalid_masks, 0)
    path = path.clone()
    predict_align_mask = path >= 0
    path[path + 1 >= (tarlen + 1)] = -1
    path[path + 1 < 0] = -1
    matchmask = torch.zeros(batch_size, tarlen + 1, prelen, device=match.device, dtype=torch.bool).scatter_(
        1, path.unsqueeze(1) + 1, 1)[:, 1:]
    oracle = tgt_tokens.gather(-1, path.clip(min=0))
    same_num = ((pred_tokens == oracle) & predict_align_mask).sum(1)
    dev = tgt_tokens.device
    ndev = dev if noise_device is None else torch.device(noise_device)
    if glance_strategy is None:
        glance_nums = torch.zeros_like(target_length)
        keep_prob = ((target_length - same_num) / target_length * context_p).unsqueeze(-1) * predict_align_mask.float()
    else:
        prob = torch.randn(oracle.shape, device=ndev, dtype=torch.float, generator=generator).to(dev)
        prob.masked_fill_(~predict_align_mask, -100)
        if glance_strategy == "cmlm":
            fraction = torch.rand(target_length.shape, device=ndev, dtype=torch.float, generator=generator).to(dev)
            glance_nums = (target_length * fraction + 0.5).to(torch.long)
        else:
            glance_nums = ((target_length - same_num) * context_p + 0.5).to(torch.long)
        prob_thresh = prob.sort(descending=True)[0].gather(-1, (glance_nums - 1).clip(min=0).unsqueeze(-1)).squeeze(-1)
        prob_thresh.masked_fill_(glance_nums == 0, 100)
        keep_prob = (prob >= prob_thresh.unsqueeze(-1)).to(prob.dtype)
    keep_word_mask = (torch.rand(prev_output_tokens.shape, device=ndev, generator=generator).to(dev) < keep_prob).bool()
    glat_prev_output_tokens = prev_output_tokens.masked_fill(keep_word_mask, 0) + oracle.masked_fill(~keep_word_mask, 0)
    return {"path": path, "matchmask": matchmask, "keep_word_mask": keep_word_mask,
            "glat_prev_output_tokens": glat_prev_output_tokens, "same_num": same_num, "glance_nums": glance_nums,
            "max_tree_lprob": -(max_tree_lprob / target_length).mean()}


def viterbi_decode(unreduced_logits, unreduced_tokens, links, output_length, left_tree_mask, pad=PAD, beta=1.0,
                   ops=_default_ops, traces_on_host=False, single_call=False):
    """Viterbi decoding glue (glat_decomposed_with_link_two_hands_tri_pcfg.py:483-502): tables, length selection with the
    ``decode_viterbibeta`` penalty, readout.  ``single_call``: the same three steps as one native call
    (``ops.pcfg_viterbi_decode``).  Returns (tokens float32 [B,maxlen], pred_length [B])."""
    if single_call:
        return ops.pcfg_viterbi_decode(unreduced_logits, links, output_length.long(), unreduced_tokens, left_tree_mask, pad, beta)
    prelen = unreduced_logits.shape[1]
    scores, R_trace, L_trace, M_trace = ops.cuda_pcfg_viterbi(unreduced_logits, links, output_length.long())
    lengths = torch.arange(prelen // 4, device=scores.device).unsqueeze(0)
    length_penalty = lengths ** beta
    scores = scores / length_penalty
    scores = scores.masked_fill(scores.isnan(), float("-inf"))
    _, pred_length = torch.max(scores[:, 1:], dim=-1)
    pred_length = pred_length + 1
    if traces_on_host:  # what the reference does (:500)
        R_trace, L_trace, M_trace = R_trace.cpu(), L_trace.cpu(), M_trace.cpu()
    tokens = ops.viterbi_decoding(pred_length.long(), output_length.long(), L_trace.long(), R_trace.long(),
                                  M_trace.long(), unreduced_tokens.long(), left_tree_mask.long(), pad)
    return tokens.to(device=pred_length.device), pred_length


def decode_from_logits(logits, links, output_length, left_tree_mask, pad=PAD, beta=1.0, ops=_default_ops, single_call=False):
    """The decode from the vocabulary logits, as the model runs it (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416,
    483-502): ``log_softmax`` and ``max`` over the vocabulary, then ``viterbi_decode``.  ``single_call``: both enqueued by
    one native call (``ops.pcfg_viterbi_decode_logits``).  Returns (tokens float32 [B,maxlen], pred_length [B])."""
    if single_call:
        return ops.pcfg_viterbi_decode_logits(logits, links, output_length.long(), left_tree_mask, pad, beta)
    ob, tok = ops.logsoftmax_max(logits)
    return viterbi_decode(ob, tok, links, output_length, left_tree_mask, pad, beta, ops=ops, single_call=True)


def train_step_direct(logits, targets, links, output_length, target_length, ops=_default_ops, mark=None):
    """One training pass of the structured loss issued as the bare sequence of native calls that autograd performs for
    ``compute_pcfg_loss(...)['loss'].backward()`` (nat_pcfg_loss.py:98-145 and pcfg_loss.py:55-83, 147-179), without
    autograd bookkeeping: logsoftmax_gather (in place) -> eos mask -> inside forward + eager backward -> loss ->
    gradient scaling -> logsoftmax_gather backward (in place).  ``logits`` [B,L,V] holds d loss / d logits afterwards.
    ``mark(name, phase)`` is called before (0) and after (1) each native call so that a caller can bracket them with
    events.  Returns (loss, links_grad, ll)."""
    mark = mark or (lambda name, phase: None)
    B, L, _ = logits.shape
    idx = targets.unsqueeze(1).expand(-1, L, -1)
    mark("lsg_fwd", 0)
    match = ops._logsoftmax_gather(logits, idx, True)
    mark("lsg_fwd", 1)
    match_m = eos_masked(match, output_length, target_length)
    mark("inside_fwd", 0)
    S, aux, ol, tl = ops._pcfg_loss_tables(match_m, links, output_length, target_length, 1, "cuda_pcfg_loss")
    mark("inside_fwd", 1)
    ones = torch.ones((B,), dtype=S.dtype, device=S.device)
    mark("inside_bwd", 0)
    mg, lg = ops._pcfg_loss_backward(ones, S, aux, match_m, links, ol, tl, 1)
    mark("inside_bwd", 1)
    ll = S[:, 0, 0]
    invalid = ll.isinf().logical_or(ll.isnan())
    loss = -(ll.masked_fill(invalid, 0) / target_length).mean()
    coef = (-1.0 / (target_length * B)).to(mg.dtype).masked_fill(invalid, 0)
    gmatch = mg * coef.view(B, 1, 1)
    glinks = lg * coef.view(B, 1, 1, 1)
    mark("lsg_bwd", 0)
    ops._logsoftmax_gather_backward(logits, idx, gmatch)
    mark("lsg_bwd", 1)
    return loss, glinks, ll


def train_step_fused(logits, targets, links, output_length, target_length, ops=_default_ops, mark=None):
    """The same training pass as ``train_step_direct`` with the criterion's glue folded into the kernels: the eos mask is
    applied inside the gather (no [B,L,T] mask tensors), and the inside backward is seeded with the criterion's own
    weights -1/(n_b*B) instead of ones followed by two scaling passes; sentences with a non-finite log-likelihood get
    zero gradients from the kernel itself; the gather forward only reads the logits and the gather backward recomputes
    the softmax from the row log-sum-exps (three passes over the logits instead of four).  Four kernel launches.
    Returns (loss, links_grad, ll)."""
    mark = mark or (lambda name, phase: None)
    L = logits.shape[1]
    idx = targets.unsqueeze(1).expand(-1, L, -1)
    mark("lsg_fwd", 0)
    match_m, row_lse = ops._logsoftmax_gather_lse(logits, idx, eos_lengths=(output_length, target_length))
    mark("lsg_fwd", 1)
    mark("inside_fwd", 0)
    S, aux, ol, tl = ops._pcfg_loss_tables(match_m, links, output_length, target_length, 1, "cuda_pcfg_loss")
    mark("inside_fwd", 1)
    mark("inside_bwd", 0)
    gmatch, glinks = ops._pcfg_loss_backward(None, S, aux, match_m, links, ol, tl, 1)
    mark("inside_bwd", 1)
    mark("lsg_bwd", 0)
    ops._logsoftmax_gather_backward_lse(logits, idx, gmatch, row_lse)
    mark("lsg_bwd", 1)
    ll = S[:, 0, 0]
    invalid = ll.isinf().logical_or(ll.isnan())
    loss = -(ll.masked_fill(invalid, 0) / target_length).mean()
    return loss, glinks, ll


def train_step_single_call(logits, targets, links, output_length, target_length, ops=_default_ops, mark=None,
                           matchmask=None, keep_word_mask=None, loss_scale=1.0):
    """``train_step_fused`` issued as one native call (``pcfgnat_criterion_step``): the kernels are enqueued back to
    back by the library and the scalar loss is reduced on the device.  Returns (loss, links_grad, ll)."""
    events = None
    if mark is not None:
        events = mark("events", 6)  # the caller hands out six timing events for this step
    out, glinks, ll, _, _ = ops.pcfg_criterion_step(logits, targets, links, output_length, target_length, events=events,
                                                 matchmask=matchmask, keep_word_mask=keep_word_mask,
                                                 loss_scale=loss_scale)
    return out[0], glinks, ll
