"""TEST INFRASTRUCTURE: the five operators over the CPU oracle, with the same signatures as ``pcfg_nat_amd.custom_ops``,
so that the harness glue can be run unchanged over the oracle (CPU tensors) and compared with the HIP path."""
import numpy as np
import torch
from torch.autograd import Function

from oracle import oracle

# What the oracle has met in its arg-max decisions since the last reset_margins(), per operator: [smallest gap between the
# best and the second-best candidate (0 = an exact tie), number of exact ties, smallest gap that is not a tie] - how far
# the bit-exact index comparisons sit from a rounding flip, and how often only the scan order decides.
margins = {}


def reset_margins():
    margins["best_tree"] = [float("inf"), 0, float("inf")]
    margins["viterbi"] = [float("inf"), 0, float("inf")]


def _note(op, margin):
    if len(margin):
        m = margins[op]
        m[0] = min(m[0], float(margin[:, 0].min()))
        m[1] += int(margin[:, 1].sum())
        m[2] = min(m[2], float(margin[:, 2].min()))


def margin_text(op):
    m = margins[op]
    return "smallest arg-max margin %.3e, %d exact ties (decided by the scan order), smallest margin that is not a tie %.3e" % (
        m[0], m[1], m[2])


reset_margins()


class _Loss(Function):
    @staticmethod
    def forward(ctx, match_all, links, output_length, target_length):
        m, lk = match_all.detach().double().numpy(), links.detach().double().numpy()
        ol, tl = output_length.numpy(), target_length.numpy()
        S, C = oracle.inside_fwd(m, lk, ol, tl)
        mg, lg = oracle.inside_bwd(np.ones(len(ol)), S, C, m, lk, ol, tl)
        ctx.save_for_backward(torch.from_numpy(mg).to(match_all.dtype), torch.from_numpy(lg).to(links.dtype))
        return torch.from_numpy(S[:, 0, 0].copy()).to(match_all.dtype)

    @staticmethod
    def backward(ctx, g):
        mg, lg = ctx.saved_tensors
        return mg * g.view(-1, 1, 1), lg * g.view(-1, 1, 1, 1), None, None


cuda_pcfg_loss = _Loss.apply


def cuda_pcfg_best_tree(match_all, links, output_length, target_length):
    m, lk = match_all.detach().double().numpy(), links.detach().double().numpy()
    ol, tl = output_length.numpy(), target_length.numpy()
    S, C = oracle.inside_fwd(m, lk, ol, tl)
    tree, margin = oracle.best_tree(S, C, m, lk, ol, tl, return_margin=True)
    _note("best_tree", margin)
    return torch.from_numpy(tree), torch.from_numpy(S[:, 0, 0].copy()).float()


def cuda_pcfg_viterbi(ob_lprob, links, output_length):
    S, R, Lt, M, margin = oracle.viterbi(ob_lprob.numpy(), links.numpy(), output_length.numpy(), dtype=np.float32,
                                         return_margin=True)
    _note("viterbi", margin)
    return torch.from_numpy(S[:, 1, :].copy()), torch.from_numpy(R), torch.from_numpy(Lt), torch.from_numpy(M)


class _Gather(Function):
    @staticmethod
    def forward(ctx, word_ins_out, select_idx):
        need = ctx.needs_input_grad[0]
        sel, probs = oracle.lsg_fwd(word_ins_out.detach().numpy(), select_idx.numpy(), want_probs=need)
        ctx.mark_dirty(word_ins_out)
        ctx.set_materialize_grads(False)
        if need:
            word_ins_out.copy_(torch.from_numpy(probs).to(word_ins_out.dtype))
            ctx.save_for_backward(word_ins_out, select_idx)
        out_dtype = torch.float64 if word_ins_out.dtype == torch.float64 else torch.float32
        return word_ins_out, torch.from_numpy(sel).to(out_dtype)

    @staticmethod
    def backward(ctx, grad_word_ins_out, grad_output):
        if not ctx.needs_input_grad[0] or grad_output is None:
            return None, None
        buf, idx = ctx.saved_tensors
        buf.mul_(grad_output.sum(-1, keepdim=True).neg_().to(buf.dtype))
        buf.scatter_add_(-1, idx, grad_output.to(buf.dtype))
        return buf, None


dag_logsoftmax_gather_inplace = _Gather.apply


def viterbi_decoding(pred_length, output_length, L_trace, R_trace, M_trace, unreduced_tokens, left_tree_mask, pad_index):
    out = oracle.viterbi_decoding(pred_length.numpy(), output_length.numpy(), L_trace.numpy(), R_trace.numpy(),
                                  M_trace.numpy(), unreduced_tokens.numpy(), left_tree_mask.numpy(), int(pad_index))
    return torch.from_numpy(out)
