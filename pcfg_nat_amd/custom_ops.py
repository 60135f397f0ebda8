"""Operator API of the structured-loss path, signature-compatible with the reference's
``fs_plugins/custom_ops/pcfg_loss.py`` (exports of ``fs_plugins/custom_ops/__init__.py:1``):

    cuda_pcfg_loss, cuda_pcfg_best_tree, cuda_pcfg_viterbi, dag_logsoftmax_gather_inplace, viterbi_decoding

The autograd Functions keep the reference's names, argument order, class attributes, return order and in-place
contract; the arithmetic runs in hand-written HIP kernels for gfx950 reached through the C-ABI of
``libpcfg_nat_hip.so`` on the current HIP stream.  There is no CPU path: calling with CPU tensors (other than
``viterbi_decoding``, whose reference version is itself a host loop) raises.
"""
import contextlib
import ctypes
import threading
import time

import torch
from torch.autograd import Function

from . import _lib

_DTYPE_CODE = {torch.float16: _lib.F16, torch.float32: _lib.F32, torch.float64: _lib.F64}


def get_pcfg_kernel():
    """Loader with the reference's name (pcfg_loss.py:18-47).  Returns the ctypes library handle."""
    if not torch.cuda.is_available():
        raise RuntimeError("You need GPU to use the custom cuda operations")
    return _lib.load()


# Host side of the three training operators (cuda_pcfg_loss, dag_logsoftmax_gather_inplace, pcfg_criterion): the torch
# extension (C++ checks, allocation and autograd nodes; what a training run uses) or the Python Functions of this module
# over ctypes (same kernels, same results; kept for float64 tables and as the readable statement of the contract).
_HOST_BACKEND = "extension"


def host_backend(name=None):
    """Selects ("extension" / "python") or reports which host-side implementation the training operators use."""
    global _HOST_BACKEND
    if name is not None:
        if name not in ("extension", "python"):
            raise RuntimeError("host_backend: 'extension' or 'python'")
        _HOST_BACKEND = name
    return _HOST_BACKEND


def _ext():
    return _lib.load_ext() if _HOST_BACKEND == "extension" else None


DEFAULT_SPIN_LIMIT = 1 << 15  # PCFGNAT_DEFAULT_SPIN_LIMIT of the library


def pipeline_config(max_workgroups=None, spin_limit=None, outside_spin_limit=None):
    """Tuning of the long-graph inside sweeps (no counterpart in the reference): graphs of 130..1026 nodes are swept by
    one workgroup per block of 16 main-chain nodes, pipelined, while the batch needs no more than ``max_workgroups`` of
    them (default 2**20; 0 = always one workgroup per sentence).  ``spin_limit`` bounds the wait of a block for the one
    ahead of it (default 2**15 rounds of polling, tens of milliseconds); a sentence whose blocks give up is redone by the
    one-workgroup sweep in the same call.  ``outside_spin_limit``: a limit of its own for the outside pipeline where the
    two run side by side (negative = the common one).  ``None`` leaves a setting as it is.  The settings are process-wide
    (every thread, stream and device): for tests and tuning, not for per-call use."""
    lib = _lib.load()
    lib.pcfgnat_pipeline_config(-1 if max_workgroups is None else int(max_workgroups), -1 if spin_limit is None else int(spin_limit))
    if outside_spin_limit is not None:
        lib.pcfgnat_pipeline_outside_spin_limit(int(outside_spin_limit))


def links_grad_range_limit(log2_limit=120.0):
    """Test hook (process-wide): the largest base-2 exponent a factor of the rule posteriors of long graphs may have on the
    matrix cores before its tile is recomputed term by term; ``float('-inf')`` forces the second path everywhere."""
    _lib.load().pcfgnat_links_grad_range_limit(float(log2_limit))


def pipeline_redo_counts(reset=False):
    """(inside sweeps, single-call Viterbi decodes, sentences given up) on the current device since the library was loaded
    or the last reset: sweeps and decodes that the one-workgroup kernels had to redo because a pipelined sweep gave up, and
    sentences whose second chance also ran out of its (seconds long) bound and came back with a NaN log-likelihood - an
    invalid sentence for the criterion; must stay zero.  Synchronises with the device."""
    lib = _lib.load()
    a, b, c = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    _lib.check(lib.pcfgnat_pipeline_redo_counts(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c), int(bool(reset))), lib)
    return a.value, b.value, c.value


def pipeline_redo_wait_limit(polls=-1):
    """Test hook (process-wide): bound of the outside sweep's wait for the forward sweep where both are redone, in polls of
    about a microsecond (negative: the default, 2**23); 0 makes the wait expire at once, which gives the sentence up."""
    _lib.load().pcfgnat_pipeline_redo_wait_limit(int(polls))


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_cuda(name, *tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("%s: expected tensors on the GPU, got a %s tensor" % (name, t.device.type))
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError("%s: tensors are on different devices (%s vs %s)" % (name, dev, t.device))


def _lengths(name, t, batch):
    if t.dim() != 1 or t.size(0) != batch:
        raise RuntimeError("%s: length tensor must have shape [%d], got %s" % (name, batch, tuple(t.shape)))
    if t.dtype != torch.int64:
        raise RuntimeError("%s: lengths should be long" % name)
    return t.contiguous()


def _check_pcfg_inputs(name, match_all, links, output_length, target_length):
    _need_cuda(name, match_all, links, output_length, target_length)
    if match_all.dim() != 3:
        raise RuntimeError("%s: match_all dim != 3" % name)
    if links.dim() != 4:
        raise RuntimeError("%s: links dim != 4" % name)
    B, L, T = match_all.shape
    if links.size(0) != B or links.size(1) != L or links.size(3) != L:
        raise RuntimeError("%s: links must be [bsz, prelen, max_left+1, prelen] = [%d, %d, *, %d], got %s"
                           % (name, B, L, L, tuple(links.shape)))
    if match_all.dtype != links.dtype or match_all.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("%s: match_all and links must both be float32 or both float64 (got %s, %s)"
                           % (name, match_all.dtype, links.dtype))
    return B, L, T, links.size(2) - 1


def _is_f64(t):
    """float64 tables (which the reference also dispatches, pcfg_loss.cu:395) go to the plain float64 entry points."""
    return t.dtype == torch.float64


def _pcfg_loss_tables(match_all, links, output_length, target_length, config, name):
    """pcfg_loss (pcfg_loss.cu:379-401): returns (S [B,Mc,T+2], aux)."""
    if not (1 <= config <= 4):
        raise RuntimeError("config should be 1~4")
    lib = get_pcfg_kernel()
    B, L, T, ml = _check_pcfg_inputs(name, match_all, links, output_length, target_length)
    output_length = _lengths(name, output_length, B)
    target_length = _lengths(name, target_length, B)
    Mc = (L - 2) // (ml + 1) + 1
    with torch.cuda.device(match_all.device):
        S = torch.empty((B, Mc, T + 2), dtype=match_all.dtype, device=match_all.device)
        if _is_f64(match_all):
            aux = torch.empty((max(1, lib.pcfgnat_pcfg_aux_elems_f64(B, L, T, ml)),), dtype=torch.float64, device=match_all.device)
            fn = lib.pcfgnat_pcfg_loss_f64
        else:
            aux = torch.empty((max(1, lib.pcfgnat_pcfg_aux_floats(B, L, T, ml)),), dtype=torch.float32, device=match_all.device)
            fn = lib.pcfgnat_pcfg_loss
        _lib.check(fn(match_all.data_ptr(), links.data_ptr(), output_length.data_ptr(), target_length.data_ptr(), S.data_ptr(),
                      aux.data_ptr(), B, L, T, ml, _stream(match_all)), lib)
    return S, aux, output_length, target_length


def _pcfg_loss_backward(grad_output, S, aux, match_all, links, output_length, target_length, config):
    """pcfg_loss_backward (pcfg_loss_backward.cu:654-721).  ``grad_output=None`` selects the criterion's own weights
    -1/(target_length*B), the gradient of ``-(ll/target_length).mean()`` (nat_pcfg_loss.py:135)."""
    if not (1 <= config <= 4):
        raise RuntimeError("config should be 1~4")
    lib = get_pcfg_kernel()
    B, L, T = match_all.shape
    ml = links.size(2) - 1
    with torch.cuda.device(match_all.device):
        match_all_grad = torch.empty_like(match_all)
        links_grad = torch.empty_like(links)
        if _is_f64(match_all):
            if grad_output is None:
                raise RuntimeError("pcfg_loss_backward: the float64 path needs an explicit grad_output")
            fn = lib.pcfgnat_pcfg_loss_backward_f64
            grad_output = grad_output.to(torch.float64).contiguous()
        else:
            fn = lib.pcfgnat_pcfg_loss_backward
        _lib.check(fn(grad_output.data_ptr() if grad_output is not None else None, S.data_ptr(), aux.data_ptr(),
                      match_all.data_ptr(), links.data_ptr(), output_length.data_ptr(), target_length.data_ptr(),
                      match_all_grad.data_ptr(), links_grad.data_ptr(), B, L, T, ml, _stream(match_all)), lib)
    return match_all_grad, links_grad


def _pcfg_loss_forward_backward(grad_output, match_all, links, output_length, target_length, config, name):
    """pcfg_loss followed by pcfg_loss_backward (the eager pair of pcfg_loss.py:67-73) as one native call, a single launch
    when the sentence's tables fit in LDS.  Returns (S, match_all_grad, links_grad)."""
    if not (1 <= config <= 4):
        raise RuntimeError("config should be 1~4")
    lib = get_pcfg_kernel()
    B, L, T, ml = _check_pcfg_inputs(name, match_all, links, output_length, target_length)
    output_length = _lengths(name, output_length, B)
    target_length = _lengths(name, target_length, B)
    if _is_f64(match_all):  # two plain calls
        S, aux, output_length, target_length = _pcfg_loss_tables(match_all, links, output_length, target_length, config, name)
        mg, lg = _pcfg_loss_backward(grad_output, S, aux, match_all, links, output_length, target_length, config)
        return S, mg, lg
    Mc = (L - 2) // (ml + 1) + 1
    with torch.cuda.device(match_all.device):
        S = torch.empty((B, Mc, T + 2), dtype=torch.float32, device=match_all.device)
        aux = torch.empty((max(1, lib.pcfgnat_pcfg_aux_floats(B, L, T, ml)),), dtype=torch.float32, device=match_all.device)
        match_all_grad = torch.empty_like(match_all)
        links_grad = torch.empty_like(links)
        _lib.check(lib.pcfgnat_pcfg_loss_forward_backward(grad_output.data_ptr() if grad_output is not None else None,
                                                          match_all.data_ptr(), links.data_ptr(), output_length.data_ptr(),
                                                          target_length.data_ptr(), S.data_ptr(), aux.data_ptr(),
                                                          match_all_grad.data_ptr(), links_grad.data_ptr(), B, L, T, ml,
                                                          _stream(match_all)), lib)
    return S, match_all_grad, links_grad


class CUDAPCFGLossFunc(Function):
    """Inside-algorithm log-likelihood (reference: pcfg_loss.py:49-85)."""
    config = 1
    config1 = 1
    config2 = 1

    @staticmethod
    def forward(
        ctx,
        match_all,      # bsz * prelen * tarlen
        links,          # bsz * prelen * (max_left+1) * prelen
        output_length,  # bsz
        target_length,  # bsz
    ):
        batch_size = match_all.shape[0]
        require_gradient = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        match_all = match_all.contiguous()
        links = links.contiguous()
        if require_gradient:
            # like the reference (pcfg_loss.py:71-73) the backward sweep runs eagerly with a unit upstream gradient
            ones = torch.ones((batch_size,), dtype=match_all.dtype, device=match_all.device)
            S, match_all_grad, links_grad = _pcfg_loss_forward_backward(ones, match_all, links, output_length, target_length,
                                                                        CUDAPCFGLossFunc.config, "cuda_pcfg_loss")
            ctx.save_for_backward(match_all_grad, links_grad)
        else:
            S, _, _, _ = _pcfg_loss_tables(match_all, links, output_length, target_length, CUDAPCFGLossFunc.config,
                                           "cuda_pcfg_loss")
        return S[:, 0, 0].clone()

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            match_all_grad, links_grad = ctx.saved_tensors
            batch_size = match_all_grad.shape[0]
            return (match_all_grad * grad_output.view(batch_size, 1, 1),
                    links_grad * grad_output.view(batch_size, 1, 1, 1), None, None)
        return None, None, None, None


def max_left_path(max_left, L=None, T=None):
    """Which kernel family serves ``cuda_pcfg_loss`` for this ``max_left`` (= ``links.size(2) - 1``): "tuned" for the value
    of the shipped scripts and, at graph sizes and target lengths the library says it covers, for ``max_left = 3``;
    "generic" for the plain one-workgroup-per-sentence restatement."""
    ml = int(max_left)
    if ml == 1:
        return "tuned"
    if ml == 3 and L is not None and T is not None and get_pcfg_kernel().pcfgnat_max_left3_supported(int(L), int(T)):
        return "tuned"
    return "generic"


def max_left3_counts(reset=False, viterbi=False):
    """Diagnostic: (sentences served by the one-launch kernel for ``max_left = 3``, sentences it left to the plain kernels)
    on the current device since the last reset; ``viterbi``: the counters of the Viterbi tables instead of the loss."""
    a, b = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    lib = get_pcfg_kernel()
    fn = lib.pcfgnat_max_left3_viterbi_counts if viterbi else lib.pcfgnat_max_left3_counts
    _lib.check(fn(ctypes.byref(a), ctypes.byref(b), 1 if reset else 0), lib)
    return int(a.value), int(b.value)


def max_left3_tuned(on=-1):
    """Test hook: switches the one-launch kernel for ``max_left = 3`` off (0) or on (1); returns the previous setting."""
    return int(get_pcfg_kernel().pcfgnat_max_left3_tuned(int(on)))


def cuda_pcfg_loss(match_all, links, output_length, target_length):
    """``CUDAPCFGLossFunc.apply`` (pcfg_loss.py:85); float32 tables go through the C++ autograd node of the torch extension."""
    ext = _ext()
    if ext is None or match_all.dtype != torch.float32 or links.dtype != torch.float32 or not match_all.is_cuda:
        return CUDAPCFGLossFunc.apply(match_all, links, output_length, target_length)
    if not (1 <= CUDAPCFGLossFunc.config <= 4):
        raise RuntimeError("config should be 1~4")
    return ext.cuda_pcfg_loss(match_all, links, output_length, target_length)


class CUDAPCFGBestTreeFunc(Function):
    """GLAT alignment: greedy top-down trace over the inside tables (reference: pcfg_loss.py:89-117)."""
    config = 1

    @staticmethod
    def forward(
        ctx,
        match_all,      # bsz * prelen * tarlen
        links,          # bsz * prelen * (max_left+1) * prelen
        output_length,  # bsz
        target_length,  # bsz
    ):
        match_all = match_all.contiguous()
        links = links.contiguous()
        S, aux, ol, tl = _pcfg_loss_tables(match_all, links, output_length, target_length,
                                           CUDAPCFGBestTreeFunc.config, "cuda_pcfg_best_tree")
        lib = get_pcfg_kernel()
        B, L, T = match_all.shape
        ml = links.size(2) - 1
        with torch.cuda.device(match_all.device):
            tree = torch.empty((B, L), dtype=torch.int64, device=match_all.device)
            fn = lib.pcfgnat_pcfg_best_tree_f64 if _is_f64(match_all) else lib.pcfgnat_pcfg_best_tree
            _lib.check(fn(S.data_ptr(), aux.data_ptr(), match_all.data_ptr(), links.data_ptr(), ol.data_ptr(), tl.data_ptr(),
                          tree.data_ptr(), B, L, T, ml, _stream(match_all)), lib)
        ctx.mark_non_differentiable(tree)
        return tree, S[:, 0, 0].clone()

    @staticmethod
    def backward(ctx, grad_tree, grad_output):
        return None, None, None, None


cuda_pcfg_best_tree = CUDAPCFGBestTreeFunc.apply


class CUDAPCFGViterbiFunc(Function):
    """Max-product tables per output length (reference: pcfg_loss.py:119-142).  Returns (scores, R, L, M)."""
    config = 1

    @staticmethod
    def forward(
        ctx,
        ob_lprob,       # bsz * prelen
        links,          # bsz * prelen * (max_left+1) * prelen
        output_length,  # bsz
    ):
        # the reference reads CUDAPCFGBestTreeFunc.config here (pcfg_loss.py:133); kept
        if not (1 <= CUDAPCFGBestTreeFunc.config <= 4):
            raise RuntimeError("config should be 1~4")
        lib = get_pcfg_kernel()
        _need_cuda("cuda_pcfg_viterbi", ob_lprob, links, output_length)
        if ob_lprob.dim() != 2 or links.dim() != 4:
            raise RuntimeError("cuda_pcfg_viterbi: ob_lprob must be [bsz, prelen] and links [bsz, prelen, max_left+1, prelen]")
        if ob_lprob.dtype != links.dtype or ob_lprob.dtype not in (torch.float32, torch.float64):
            raise RuntimeError("cuda_pcfg_viterbi: ob_lprob and links must both be float32 or both float64 (got %s, %s)"
                               % (ob_lprob.dtype, links.dtype))
        B, L = ob_lprob.shape
        if links.size(0) != B or links.size(1) != L or links.size(3) != L:
            raise RuntimeError("cuda_pcfg_viterbi: links shape %s does not match ob_lprob %s"
                               % (tuple(links.shape), tuple(ob_lprob.shape)))
        ml = links.size(2) - 1
        ob_lprob = ob_lprob.contiguous()
        links = links.contiguous()
        output_length = _lengths("cuda_pcfg_viterbi", output_length, B)
        Lq = L // 4
        with torch.cuda.device(ob_lprob.device):
            S = torch.empty((B, L, Lq), dtype=ob_lprob.dtype, device=ob_lprob.device)
            R = torch.empty((B, L, Lq), dtype=torch.int64, device=ob_lprob.device)
            Lt = torch.empty_like(R)
            M = torch.empty_like(R)
            fn = lib.pcfgnat_pcfg_viterbi_f64 if _is_f64(ob_lprob) else lib.pcfgnat_pcfg_viterbi
            _lib.check(fn(ob_lprob.data_ptr(), links.data_ptr(), output_length.data_ptr(), S.data_ptr(), R.data_ptr(),
                          Lt.data_ptr(), M.data_ptr(), B, L, ml, _stream(ob_lprob)), lib)
        ctx.mark_non_differentiable(R, Lt, M)
        return S[:, 1, :].clone(), R, Lt, M

    @staticmethod
    def backward(ctx, *grads):
        return None, None, None


cuda_pcfg_viterbi = CUDAPCFGViterbiFunc.apply


class DagLogsoftmaxGatherFunc(Function):
    """Fused log-softmax + gather with the reference's in-place contract (pcfg_loss.py:144-181): the logits buffer is
    handed back marked dirty, must not be used by the caller any more, and becomes the gradient buffer in backward,
    which may run once.  Unlike the reference, whose forward already overwrites the buffer with softmax probabilities,
    the forward here only reads it and keeps one log-sum-exp per row; the backward recomputes the probabilities while
    it writes the gradient (three passes over the logits per step instead of four)."""

    @staticmethod
    def forward(
        ctx,
        word_ins_out,  # bsz * prelen * vocabsize
        select_idx,    # bsz * prelen * slen
    ):
        require_gradient = ctx.needs_input_grad[0]
        if require_gradient:
            selected_result, row_lse = _logsoftmax_gather_lse(word_ins_out, select_idx)
        else:
            selected_result = _logsoftmax_gather(word_ins_out, select_idx, False)
        # Note: the backward reuses word_ins_out as the gradient buffer
        ctx.mark_dirty(word_ins_out)
        ctx.set_materialize_grads(False)

        if require_gradient:
            ctx.save_for_backward(word_ins_out, select_idx, row_lse)
            ctx.has_backward = False
        return word_ins_out, selected_result  # bsz * prelen * slen

    @staticmethod
    def backward(ctx, grad_word_ins_out, grad_output):
        if not ctx.needs_input_grad[0]:
            return None, None
        assert grad_word_ins_out is None, "Cannot reuse word_ins_out after logsoftmax_gather"
        if grad_output is None:
            return None, None

        assert not ctx.has_backward, "Cannot backward twice in logsoftmax_gather"
        ctx.has_backward = True

        grad_input, selected_idx, row_lse = ctx.saved_tensors
        _logsoftmax_gather_backward_lse(grad_input, selected_idx, grad_output, row_lse)
        return grad_input, None


def dag_logsoftmax_gather_inplace(word_ins_out, select_idx):
    """``DagLogsoftmaxGatherFunc.apply`` (pcfg_loss.py:181), through the C++ autograd node of the torch extension."""
    ext = _ext()
    if ext is None or not word_ins_out.is_cuda:
        return DagLogsoftmaxGatherFunc.apply(word_ins_out, select_idx)
    return ext.dag_logsoftmax_gather_inplace(word_ins_out, select_idx)


def _logsoftmax_gather(word_ins_out, select_idx, require_gradient, eos_lengths=None):
    """logsoftmax_gather (logsoftmax_gather.cu:295-359), argument checks included (:297-309).  ``eos_lengths`` =
    (output_length, target_length) folds the criterion's eos mask (nat_pcfg_loss.py:111-115) into the gather."""
    lib = get_pcfg_kernel()
    _need_cuda("logsoftmax_gather", word_ins_out, select_idx)
    if word_ins_out.dim() != 3:
        raise RuntimeError("word_ins_out dim != 3")
    if select_idx.dim() != 3:
        raise RuntimeError("select_idx dim != 3")
    B, L, V = word_ins_out.shape
    T = select_idx.size(2)
    if select_idx.size(0) != B:
        raise RuntimeError("batch size not match")
    if select_idx.size(1) != L:
        raise RuntimeError("prelen size not match")
    if select_idx.dtype != torch.int64:
        raise RuntimeError("select_idx should be long")
    if not word_ins_out.is_contiguous():
        raise RuntimeError("word_ins_out is not contiguous")
    code = _DTYPE_CODE.get(word_ins_out.dtype)
    if code is None:
        raise RuntimeError("logsoftmax_gather: unsupported dtype %s (float16, float32, float64 are dispatched)"
                           % word_ins_out.dtype)
    out_dtype = torch.float64 if word_ins_out.dtype == torch.float64 else torch.float32
    with torch.cuda.device(word_ins_out.device):
        selected = torch.empty((B, L, T), dtype=out_dtype, device=word_ins_out.device)
        sb, sl, st = select_idx.stride()
        if eos_lengths is None:
            _lib.check(lib.pcfgnat_logsoftmax_gather(word_ins_out.data_ptr(), code, select_idx.data_ptr(), sb, sl, st,
                                                     selected.data_ptr(), int(bool(require_gradient)), B, L, V, T,
                                                     _stream(word_ins_out)), lib)
        else:
            ol = _lengths("logsoftmax_gather", eos_lengths[0], B)
            tl = _lengths("logsoftmax_gather", eos_lengths[1], B)
            _need_cuda("logsoftmax_gather", word_ins_out, ol, tl)
            _lib.check(lib.pcfgnat_logsoftmax_gather_eos(word_ins_out.data_ptr(), code, select_idx.data_ptr(), sb, sl, st,
                                                         selected.data_ptr(), int(bool(require_gradient)), ol.data_ptr(),
                                                         tl.data_ptr(), B, L, V, T, _stream(word_ins_out)), lib)
    return selected


def logsoftmax_max(logits):
    """``logits.log_softmax(-1).max(-1)`` (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-415) in one read of the
    logits: returns (best log-probability [B,L] float32 - float64 for float64 logits -, first arg max [B,L] int64)."""
    lib = get_pcfg_kernel()
    _need_cuda("logsoftmax_max", logits)
    if logits.dim() != 3 or not logits.is_contiguous():
        raise RuntimeError("logsoftmax_max: logits must be a contiguous [bsz, prelen, vocab] tensor")
    code = _DTYPE_CODE.get(logits.dtype)
    if code is None:
        raise RuntimeError("logsoftmax_max: unsupported dtype %s (float16, float32, float64 are dispatched)" % logits.dtype)
    B, L, V = logits.shape
    out_dtype = torch.float64 if logits.dtype == torch.float64 else torch.float32
    with torch.cuda.device(logits.device):
        best = torch.empty((B, L), dtype=out_dtype, device=logits.device)
        idx = torch.empty((B, L), dtype=torch.int64, device=logits.device)
        _lib.check(lib.pcfgnat_logsoftmax_max(logits.data_ptr(), code, best.data_ptr(), idx.data_ptr(), B, L, V,
                                              _stream(logits)), lib)
    return best, idx


def _logsoftmax_gather_lse(word_ins_out, select_idx, eos_lengths=None):
    """Read-only forward of the log-sum-exp split: returns (selected [B,L,T], row log-sum-exp [B,L]); same checks as
    ``_logsoftmax_gather``.  ``word_ins_out`` must stay untouched until ``_logsoftmax_gather_backward_lse`` consumes it."""
    lib = get_pcfg_kernel()
    _need_cuda("logsoftmax_gather", word_ins_out, select_idx)
    if word_ins_out.dim() != 3:
        raise RuntimeError("word_ins_out dim != 3")
    if select_idx.dim() != 3:
        raise RuntimeError("select_idx dim != 3")
    B, L, V = word_ins_out.shape
    T = select_idx.size(2)
    if select_idx.size(0) != B:
        raise RuntimeError("batch size not match")
    if select_idx.size(1) != L:
        raise RuntimeError("prelen size not match")
    if select_idx.dtype != torch.int64:
        raise RuntimeError("select_idx should be long")
    if not word_ins_out.is_contiguous():
        raise RuntimeError("word_ins_out is not contiguous")
    code = _DTYPE_CODE.get(word_ins_out.dtype)
    if code is None:
        raise RuntimeError("logsoftmax_gather: unsupported dtype %s (float16, float32, float64 are dispatched)"
                           % word_ins_out.dtype)
    out_dtype = torch.float64 if word_ins_out.dtype == torch.float64 else torch.float32
    with torch.cuda.device(word_ins_out.device):
        selected = torch.empty((B, L, T), dtype=out_dtype, device=word_ins_out.device)
        row_lse = torch.empty((B, L), dtype=out_dtype, device=word_ins_out.device)
        sb, sl, st = select_idx.stride()
        ol_ptr = tl_ptr = None
        if eos_lengths is not None:
            ol = _lengths("logsoftmax_gather", eos_lengths[0], B)
            tl = _lengths("logsoftmax_gather", eos_lengths[1], B)
            _need_cuda("logsoftmax_gather", word_ins_out, ol, tl)
            ol_ptr, tl_ptr = ol.data_ptr(), tl.data_ptr()
        _lib.check(lib.pcfgnat_logsoftmax_gather_lse(word_ins_out.data_ptr(), code, select_idx.data_ptr(), sb, sl, st,
                                                     selected.data_ptr(), row_lse.data_ptr(), ol_ptr, tl_ptr, B, L, V, T,
                                                     _stream(word_ins_out)), lib)
    return selected, row_lse


def _logsoftmax_gather_backward_lse(buf, select_idx, grad_output, row_lse):
    """In place: ``buf`` (the untouched logits) becomes d/d logits of sum(grad_output * selected): one pass that
    recomputes exp(x - lse), scales by -(sum g) and adds g at the gathered columns, rounded to buf's dtype once."""
    lib = get_pcfg_kernel()
    B, L, V = buf.shape
    T = select_idx.size(2)
    want = torch.float64 if buf.dtype == torch.float64 else torch.float32
    g = grad_output.to(want).contiguous()
    if row_lse.dtype != want or row_lse.shape != (B, L) or not row_lse.is_contiguous():
        raise RuntimeError("logsoftmax_gather_backward: row_lse must be a contiguous [bsz, prelen] tensor of %s" % want)
    with torch.cuda.device(buf.device):
        sb, sl, st = select_idx.stride()
        _lib.check(lib.pcfgnat_logsoftmax_gather_backward_lse(buf.data_ptr(), _DTYPE_CODE[buf.dtype], select_idx.data_ptr(),
                                                              sb, sl, st, g.data_ptr(), row_lse.data_ptr(), B, L, V, T,
                                                              _stream(buf)), lib)
    return buf


def _logsoftmax_gather_backward(buf, select_idx, grad_output):
    """One fused pass for ``buf.mul_(-(sum g).to(dtype)); buf.scatter_add_(-1, idx, g.to(dtype))`` (pcfg_loss.py:176-177)."""
    lib = get_pcfg_kernel()
    B, L, V = buf.shape
    T = select_idx.size(2)
    want = torch.float64 if buf.dtype == torch.float64 else torch.float32
    g = grad_output.to(want).contiguous()
    with torch.cuda.device(buf.device):
        sb, sl, st = select_idx.stride()
        _lib.check(lib.pcfgnat_logsoftmax_gather_backward(buf.data_ptr(), _DTYPE_CODE[buf.dtype], select_idx.data_ptr(),
                                                          sb, sl, st, g.data_ptr(), B, L, V, T, _stream(buf)), lib)
    return buf


def viterbi_decoding(pred_length, output_length, L_trace, R_trace, M_trace, unreduced_tokens, left_tree_mask, pad_index):
    """Tree-to-sequence readout (reference: pcfg_loss.py:183-184 -> pcfg_loss.cpp:12-73).

    Walks the (L, R, M) back-pointers from (node 1, pred_length) in order, emitting ``unreduced_tokens[node]`` unless
    it is the pad symbol or repeats the previous emission.  Returns float32 ``[B, maxlen]`` right-padded with
    ``pad_index`` (the reference's dtype, :65; it can only assemble rows of equal length, ragged batches get the
    evidently intended padding).  Traces on the GPU are walked on the GPU (one thread per sentence); CPU tensors, which
    is what the reference's caller passes, are walked by the library's host routine.
    """
    lib = _lib.load()
    B, L, Lq = L_trace.shape
    tensors = [pred_length, output_length, L_trace, R_trace, M_trace, unreduced_tokens, left_tree_mask]
    dev = L_trace.device
    args = [t.to(device=dev, dtype=torch.int64).contiguous() for t in tensors]
    pl, ol, Lt, Rt, Mt, tok, mask = args
    if mask.dim() != 2 or mask.size(0) != mask.size(1):
        raise RuntimeError("viterbi_decoding: left_tree_mask must be square")
    out = torch.empty((B, L), dtype=torch.int64, device=dev)
    if dev.type == "cuda":
        with torch.cuda.device(dev):
            scratch = torch.empty((B, 2 * L), dtype=torch.int64, device=dev)
            cnt = _pinned_counts.take(B)  # written by the kernel, read after the one stream wait
            try:
                armed = _pinned_counts.arm(cnt, B, torch.cuda.current_stream(dev))
                _lib.check(lib.pcfgnat_viterbi_decoding(pl.data_ptr(), ol.data_ptr(), Lt.data_ptr(), Rt.data_ptr(), Mt.data_ptr(),
                                                        tok.data_ptr(), mask.data_ptr(), mask.size(0), int(pad_index),
                                                        out.data_ptr(), cnt.data_ptr(), scratch.data_ptr(), B, L, Lq,
                                                        _stream(out)), lib)
                counts = _pinned_counts.wait(cnt, B, torch.cuda.current_stream(dev), armed)
            finally:
                _pinned_counts.give_back(cnt)
    else:
        cnt = torch.empty((B,), dtype=torch.int64)
        _lib.check(lib.pcfgnat_viterbi_decoding_host(pl.data_ptr(), ol.data_ptr(), Lt.data_ptr(), Rt.data_ptr(),
                                                     Mt.data_ptr(), tok.data_ptr(), mask.data_ptr(), mask.size(0),
                                                     int(pad_index), out.data_ptr(), cnt.data_ptr(), B, L, Lq), lib)
        counts = cnt.tolist()
    if B and min(counts) < 0:
        raise RuntimeError("viterbi_decoding: malformed traces")
    maxlen = max(counts) if B else 0
    return out[:, :maxlen].to(torch.float32)


_MASK_CACHE = {}


def _as_flag_mask(t):
    """A support mask as the kernels read it (one byte per entry, non-zero = set).  The masks of a model are built once per
    graph length and handed to every call, often as fresh views of one tensor (``mask[:L, :L]``): the converted copy of an
    integer mask is kept under the view's storage address, offset, shape, strides and version counter, together with the
    tensor it was made from (which keeps that storage, and with it the address, from being reused), so that a call does not
    pay a launch per mask.  Tensors without a version counter (created under ``torch.inference_mode``) are converted on
    every call."""
    if t.dtype in (torch.bool, torch.uint8):
        return t.contiguous()
    try:
        version = t._version
    except RuntimeError:  # inference tensors do not track versions
        return t.ne(0).contiguous()
    key = (t.untyped_storage().data_ptr(), t.storage_offset(), version, t.dtype, tuple(t.shape), tuple(t.stride()), str(t.device))
    hit = _MASK_CACHE.get(key)
    if hit is not None:
        return hit[1]
    flags = t.ne(0).contiguous()
    if len(_MASK_CACHE) >= 64:
        _MASK_CACHE.clear()
    _MASK_CACHE[key] = (t, flags)
    return flags


class PCFGExtractLinksFunc(Function):
    """The model's link scorer after its projections (glat_decomposed_with_link_two_hands_tri_pcfg.py:153-199).  For fp16
    and fp32 chunks with head dimensions the library covers, the batched products run on the matrix cores inside the
    kernels (one launch forward, three backward).  Otherwise (float64, other head dimensions) the products go through
    torch's GEMM library (one product forward, two backward) and everything else (packing, masking, the gather of the
    left terms, the joint log-softmax over (left option, right child) per head, the gate mixture and the whole backward of
    these) runs in five small kernels.  Neither form materialises a [B,L,2L,H] tensor."""

    @staticmethod
    def forward(ctx, query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad_index,
                left_tree_mask, right_tree_mask, main_chain, products_inside=True):
        lib = get_pcfg_kernel()
        _need_cuda("pcfg_extract_links", query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens,
                   left_tree_mask, right_tree_mask, main_chain)
        if query_chunks.dim() != 4 or key_chunks_left.shape != query_chunks.shape or key_chunks_right.shape != query_chunks.shape:
            raise RuntimeError("pcfg_extract_links: query and key chunks must share the shape [bsz, prelen, heads, head_dim]")
        if not (query_chunks.dtype == key_chunks_left.dtype == key_chunks_right.dtype) or query_chunks.dtype not in _DTYPE_CODE:
            raise RuntimeError("pcfg_extract_links: query and key chunks must share one of float16, float32, float64")
        B, L, H, F = query_chunks.shape
        if gate_logits.shape != (B, L, H) or prev_output_tokens.shape != (B, L):
            raise RuntimeError("pcfg_extract_links: gate_logits must be [bsz, prelen, heads] and prev_output_tokens [bsz, prelen]")
        if left_tree_mask.shape != (L, L) or right_tree_mask.shape != (L, L) or main_chain.shape != (L,):
            raise RuntimeError("pcfg_extract_links: tree masks must be [prelen, prelen] and main_chain [prelen]")
        dev = query_chunks.device
        code = _DTYPE_CODE[query_chunks.dtype]
        fused = products_inside and bool(lib.pcfgnat_extract_links_fused_supported(code, L, H, F))
        with torch.cuda.device(dev):
            st = _stream(query_chunks)
            q, kl, kr = query_chunks.contiguous(), key_chunks_left.contiguous(), key_chunks_right.contiguous()
            # what the kernels with the products inside also ask for: chunks on 16-byte boundaries (a contiguous view at
            # an odd storage offset is not) and, in the backward, a batch that fits its grid; otherwise the five-call
            # form, which takes any layout
            fused = fused and all(x.data_ptr() % 16 == 0 for x in (q, kl, kr)) and B <= 32767
            fused_bwd = bool(lib.pcfgnat_extract_links_fused_backward_supported(code, L, H, F))
            need_grad = any(ctx.needs_input_grad[:4])
            ctx.fused = fused and (fused_bwd or not need_grad)
            if ctx.fused:
                # the products on the matrix cores inside the kernels: one launch forward, three backward
                gate = gate_logits.float().contiguous()
                prev = prev_output_tokens.to(torch.int64).contiguous()
                masks = [_as_flag_mask(t) for t in (left_tree_mask, right_tree_mask, main_chain)]
                links = torch.empty((B, L, 2, L), dtype=torch.float32, device=dev)
                # the per-head normalisers and, for the backward, the masks per parent as bits: one allocation
                nw = 1 + (L + 31) // 32
                side = torch.empty((B * L * (H + (nw if need_grad else 0)),), dtype=torch.float32, device=dev)
                lse = side[:B * L * H].view(B, L, H)
                tile_masks = side[B * L * H:].view(torch.int32).view(B, L, nw) if need_grad else None
                _lib.check(lib.pcfgnat_extract_links_fused_forward(q.data_ptr(), kl.data_ptr(), kr.data_ptr(), code, gate.data_ptr(),
                                                                   prev.data_ptr(), int(pad_index), masks[0].data_ptr(),
                                                                   masks[1].data_ptr(), masks[2].data_ptr(), links.data_ptr(),
                                                                   lse.data_ptr(), tile_masks.data_ptr() if need_grad else None,
                                                                   B, L, H, F, st), lib)
                if need_grad:
                    ctx.save_for_backward(links, lse, tile_masks, q, kl, kr, gate)
                    ctx.chunk_dtype, ctx.gate_dtype = query_chunks.dtype, gate_logits.dtype
                return links
            A = torch.empty((B, H, 2 * L, F), dtype=torch.float32, device=dev)
            Kr = torch.empty((B, H, L, F), dtype=torch.float32, device=dev)
            _lib.check(lib.pcfgnat_extract_links_pack(q.data_ptr(), kl.data_ptr(), kr.data_ptr(), code, A.data_ptr(), Kr.data_ptr(),
                                                      B, L, H, F, st), lib)
            Z = torch.matmul(A, Kr.transpose(-1, -2))
            gate = gate_logits.float().contiguous()
            prev = prev_output_tokens.to(torch.int64).contiguous()
            masks = [_as_flag_mask(t) for t in (left_tree_mask, right_tree_mask, main_chain)]
            links = torch.empty((B, L, 2, L), dtype=torch.float32, device=dev)
            lse = torch.empty((B, L, H), dtype=torch.float32, device=dev)
            _lib.check(lib.pcfgnat_extract_links_forward(Z.data_ptr(), A.data_ptr(), gate.data_ptr(), prev.data_ptr(), int(pad_index),
                                                         masks[0].data_ptr(), masks[1].data_ptr(), masks[2].data_ptr(),
                                                         links.data_ptr(), lse.data_ptr(), B, L, H, F, st), lib)
        ctx.save_for_backward(links, lse, Z, A, Kr, gate, prev, *masks)
        ctx.fused = False
        ctx.pad_index = int(pad_index)
        ctx.chunk_dtype, ctx.gate_dtype = query_chunks.dtype, gate_logits.dtype
        return links

    @staticmethod
    def backward(ctx, grad_links):
        lib = get_pcfg_kernel()
        if ctx.fused:
            links, lse, tile_masks, q, kl, kr, gate = ctx.saved_tensors
            B, L, H, F = q.shape
            dev = q.device
            code = _DTYPE_CODE[ctx.chunk_dtype]
            with torch.cuda.device(dev):
                st = _stream(q)
                G = grad_links.float().contiguous()
                if G.data_ptr() % 16:  # (a view at an odd offset: the kernels read it in 16-byte pieces)
                    G = G.clone()
                dq, dkl, dkr = torch.empty((3, B, L, H, F), dtype=q.dtype, device=dev).unbind(0)  # one allocation each way
                nws = (lib.pcfgnat_extract_links_fused_backward_workspace_bytes(B, L, H, F) + 3) // 4
                block = torch.empty((nws + B * L * H,), dtype=torch.float32, device=dev)  # the workspace first: it wants 16-byte alignment
                ws, dgate = block[:nws], block[nws:].view(B, L, H)
                _lib.check(lib.pcfgnat_extract_links_fused_backward(G.data_ptr(), links.data_ptr(), lse.data_ptr(), tile_masks.data_ptr(),
                                                                    q.data_ptr(), kl.data_ptr(), kr.data_ptr(), code, gate.data_ptr(),
                                                                    dq.data_ptr(), dkl.data_ptr(), dkr.data_ptr(), dgate.data_ptr(),
                                                                    ws.data_ptr(), B, L, H, F, st), lib)
            return dq, dkl, dkr, dgate.to(ctx.gate_dtype), None, None, None, None, None, None
        links, lse, Z, A, Kr, gate, prev, ltm, rtm, mc = ctx.saved_tensors
        B, H, L2, F = A.shape
        L = L2 // 2
        dev = A.device
        with torch.cuda.device(dev):
            st = _stream(A)
            G = grad_links.float().contiguous()
            dZ = torch.empty_like(Z)
            dZ0 = torch.empty((B, H, L, L), dtype=torch.float32, device=dev)
            dsab = torch.empty((B, H, L, 2), dtype=torch.float32, device=dev)
            dgate = torch.empty((B, L, H), dtype=torch.float32, device=dev)
            _lib.check(lib.pcfgnat_extract_links_backward(G.data_ptr(), links.data_ptr(), lse.data_ptr(), Z.data_ptr(), A.data_ptr(),
                                                          gate.data_ptr(), prev.data_ptr(), ctx.pad_index, ltm.data_ptr(), rtm.data_ptr(),
                                                          mc.data_ptr(), dZ.data_ptr(), dZ0.data_ptr(), dsab.data_ptr(), dgate.data_ptr(),
                                                          B, L, H, F, st), lib)
            dA = torch.matmul(dZ, Kr)
            dKr = torch.matmul(dZ.transpose(-1, -2), A)
            dq = torch.empty((B, L, H, F), dtype=ctx.chunk_dtype, device=dev)
            dkl, dkr = torch.empty_like(dq), torch.empty_like(dq)
            _lib.check(lib.pcfgnat_extract_links_unpack(dA.data_ptr(), dKr.data_ptr(), dsab.data_ptr(), A.data_ptr(),
                                                        _DTYPE_CODE[ctx.chunk_dtype], dq.data_ptr(), dkl.data_ptr(), dkr.data_ptr(),
                                                        B, L, H, F, st), lib)
        return dq, dkl, dkr, dgate.to(ctx.gate_dtype), None, None, None, None, None, None


def pcfg_extract_links(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad_index, left_tree_mask,
                       right_tree_mask, main_chain, products_inside=True):
    """links [bsz, prelen, 2, prelen] float32 from the projected chunks [bsz, prelen, heads, head_dim] and the gate logits
    [bsz, prelen, heads]; differentiable in the first four arguments.  max_left = 1.  products_inside=False takes the form
    whose products go through torch's GEMM library also where the library's own kernels would cover the shape."""
    ext = _ext()
    if (ext is not None and products_inside and query_chunks.is_cuda and query_chunks.dim() == 4
            and query_chunks.dtype in (torch.float16, torch.float32) and query_chunks.size(0) <= 32767):
        # the C++ autograd node, where the kernels with the products inside cover the shape and the layout
        lib = get_pcfg_kernel()
        code = _DTYPE_CODE[query_chunks.dtype]
        _, L, H, F = query_chunks.shape
        need_grad = any(t.requires_grad for t in (query_chunks, key_chunks_left, key_chunks_right, gate_logits))
        if (lib.pcfgnat_extract_links_fused_supported(code, L, H, F)
                and (not need_grad or lib.pcfgnat_extract_links_fused_backward_supported(code, L, H, F))
                and all(t.is_contiguous() and t.data_ptr() % 16 == 0 for t in (query_chunks, key_chunks_left, key_chunks_right))):
            masks = [_as_flag_mask(t) for t in (left_tree_mask, right_tree_mask, main_chain)]
            masks = [m.view(torch.uint8) if m.dtype == torch.bool else m for m in masks]  # (same bytes)
            return ext.pcfg_extract_links_fused(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens,
                                                int(pad_index), *masks)
    return PCFGExtractLinksFunc.apply(query_chunks, key_chunks_left, key_chunks_right, gate_logits, prev_output_tokens, pad_index,
                                      left_tree_mask, right_tree_mask, main_chain, products_inside)


GLANCE_STRATEGIES = {"number-random": 0, "cmlm": 1, None: 2}  # PCFGNAT_GLANCE_* of the library


def pcfg_glat_step(word_ins_out, tgt_tokens, prev_output_tokens, links, context_p, pad_index, generator=None,
                   noise_device=None, glance_strategy="number-random"):
    """GLAT glancing (nat_pcfg_loss.py:193-269) as one native call, for each glance strategy of the reference
    (``"number-random"``, ``"cmlm"``, ``None``).  Same results as the torch glue over the separate ops; ``word_ins_out``
    is only read.  The random draws of the reference (``randn`` for the glance scores, ``rand`` for cmlm's lengths, then
    ``rand`` for the revealed nodes, as far as the strategy makes them) are made here, in that order, on the tokens' device
    or on ``noise_device``.  Returns the dict of ``harness.glat_alignment``."""
    if glance_strategy not in GLANCE_STRATEGIES:
        raise RuntimeError("pcfg_glat_step: unknown glance strategy %r" % (glance_strategy,))
    lib = get_pcfg_kernel()
    _need_cuda("pcfg_glat_step", word_ins_out, tgt_tokens, prev_output_tokens, links)
    if word_ins_out.dim() != 3 or not word_ins_out.is_contiguous():
        raise RuntimeError("pcfg_glat_step: word_ins_out must be a contiguous [bsz, prelen, vocab] tensor")
    B, L, V = word_ins_out.shape
    code = _DTYPE_CODE.get(word_ins_out.dtype)
    if code is None:
        raise RuntimeError("pcfg_glat_step: unsupported dtype %s" % word_ins_out.dtype)
    if tgt_tokens.dim() != 2 or tgt_tokens.size(0) != B or tgt_tokens.dtype != torch.int64:
        raise RuntimeError("pcfg_glat_step: tgt_tokens must be an int64 [bsz, tarlen] tensor")
    if prev_output_tokens.shape != (B, L) or prev_output_tokens.dtype != torch.int64:
        raise RuntimeError("pcfg_glat_step: prev_output_tokens must be an int64 [bsz, prelen] tensor")
    if links.dim() != 4 or links.size(0) != B or links.size(1) != L or links.size(3) != L or links.dtype != torch.float32:
        raise RuntimeError("pcfg_glat_step: links must be float32 [bsz, prelen, max_left+1, prelen]")
    T = tgt_tokens.size(1)
    ml = links.size(2) - 1
    Mc = (L - 2) // (ml + 1) + 1
    dev = word_ins_out.device
    tgt, prev, links = tgt_tokens.contiguous(), prev_output_tokens.contiguous(), links.contiguous()
    ndev = dev if noise_device is None else torch.device(noise_device)
    noise = len_rand = keep_rand = None
    if glance_strategy is not None:
        noise = torch.randn((B, L), device=ndev, dtype=torch.float, generator=generator).to(dev)
    if glance_strategy == "cmlm":
        len_rand = torch.rand((B,), device=ndev, dtype=torch.float, generator=generator).to(dev)
    keep_rand = torch.rand((B, L), device=ndev, generator=generator)  # the reference's last draw
    # (number-random, cmlm: it cannot change the result and is made only to keep the stream in step)
    keep_rand = keep_rand.to(dev) if glance_strategy is None else None
    with torch.cuda.device(dev):
        f32 = dict(dtype=torch.float32, device=dev)
        i64 = dict(dtype=torch.int64, device=dev)
        match = torch.empty((B, L, T), **f32)
        S = torch.empty((B, Mc, T + 2), **f32)
        aux = torch.empty((max(1, lib.pcfgnat_pcfg_aux_floats(B, L, T, ml)),), **f32)
        ints = torch.empty((4, B, L), **i64)       # pred_tokens, path, glat tokens, (unused)
        small = torch.empty((4, B), **i64)         # output_length, target_length, same_num, glance_nums
        matchmask = torch.empty((B, T, L), dtype=torch.bool, device=dev)
        keep = torch.empty((B, L), dtype=torch.bool, device=dev)
        out = torch.empty((2,), **f32)
        ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
        _lib.check(lib.pcfgnat_glat_step(word_ins_out.data_ptr(), code, tgt.data_ptr(), prev.data_ptr(), links.data_ptr(),
                                         GLANCE_STRATEGIES[glance_strategy], ptr(noise), ptr(len_rand), ptr(keep_rand),
                                         float(context_p), int(pad_index), match.data_ptr(), S.data_ptr(),
                                         aux.data_ptr(), ints[0].data_ptr(), small[0].data_ptr(), ints[1].data_ptr(),
                                         matchmask.data_ptr(), keep.data_ptr(), ints[2].data_ptr(), small[2].data_ptr(),
                                         small[3].data_ptr(), out.data_ptr(), B, L, V, T, ml, _stream(word_ins_out)), lib)
    return {"path": ints[1], "matchmask": matchmask, "keep_word_mask": keep, "glat_prev_output_tokens": ints[2],
            "same_num": small[2], "glance_nums": small[3], "max_tree_lprob": out[0]}


_PENALTY_CACHE = {}


def _length_penalty(Lq, beta, device):
    """``arange(Lq) ** beta`` as the reference computes it (glat_decomposed_with_link_two_hands_tri_pcfg.py:489-492),
    cached per (Lq, beta, device)."""
    key = (int(Lq), float(beta), device.type, device.index)
    pen = _PENALTY_CACHE.get(key)
    if pen is None:
        pen = (torch.arange(Lq).unsqueeze(0) ** beta).to(device=device, dtype=torch.float32).contiguous().view(-1)
        _PENALTY_CACHE[key] = pen
    return pen


class _CountBuffer:
    """One pinned int64 host buffer: the tensor that owns the memory, its address, and the same words as a ctypes array
    (the host marks and reads a handful of entries per call; going through the array costs a fraction of a tensor op)."""
    __slots__ = ("tensor", "ptr", "words", "capacity")

    def __init__(self, n):
        self.capacity = max(n, 64)
        self.tensor = torch.empty((self.capacity,), dtype=torch.int64, pin_memory=True)
        self.ptr = self.tensor.data_ptr()
        self.words = (ctypes.c_int64 * self.capacity).from_address(self.ptr)

    def data_ptr(self):
        return self.ptr


class _PinnedCounts:
    """Pinned int64 host buffers for the per-sentence token counts of the decode calls.  Pinned host memory is addressable
    from the device, so the kernels write the counts straight into it and the caller reads them as they arrive (``arm`` /
    ``wait`` below), at the latest after waiting for its stream.  A call takes a buffer out of the pool for its own use and
    puts it back when it has read the counts: calls that overlap (several host threads, several streams of one device)
    never share one.  Allocating pinned memory takes about a hundred microseconds, hence the pool; it holds as many buffers
    as calls have ever overlapped."""

    def __init__(self):
        self._lock = threading.Lock()
        self._free = []
        self._polling = True
        self._misses = 0

    def take(self, n):
        with self._lock:
            for i, buf in enumerate(self._free):
                if buf.capacity >= n:
                    return self._free.pop(i)
        return _CountBuffer(n)

    def give_back(self, buf):
        with self._lock:
            self._free.append(buf)

    # The kernels write a sentence's count (>= -1) as the last thing they do for it.  Instead of waiting for the stream,
    # whose wake-up costs the host some microseconds after the kernel has ended, the caller marks the entries before the
    # launch and watches them turn: device stores to pinned host memory reach the host while the kernel is still running.
    # The watch is for the latency-bound case only - a decode enqueued on an idle stream: with work already pending on the
    # stream (``stream.query()`` false before the launch) the call goes straight to the stream wait.  A watch is bounded by
    # time; one that runs into its bound hands over to the stream wait for that call, and only after several such misses
    # in a row (a host-memory mode in which the stores only arrive with the end of the kernel) is the watching switched off.
    NOT_YET = -2
    WATCH_SECONDS = 0.005       # longest a call watches before it waits for the stream instead
    MISSES_TO_SWITCH_OFF = 8    # consecutive watches that ran into the bound

    def polling_on(self):
        return self._polling

    def arm(self, buf, n, stream):
        """Marks the entries and returns True if this call is going to watch them."""
        if not self._polling or not stream.query():
            return False
        words = buf.words
        for i in range(n):
            words[i] = self.NOT_YET
        return True

    def wait(self, buf, n, stream, armed):
        """Returns the n counts once the kernels have written them.  ``stream``: the stream of the call, or a device (its
        current stream is looked up only if the call has to wait for it)."""
        words = buf.words
        if armed:
            not_yet = self.NOT_YET
            deadline = time.perf_counter() + self.WATCH_SECONDS
            i = spins = 0
            while i < n:
                if words[i] != not_yet:
                    i += 1
                    continue
                spins += 1
                if (spins & 255) == 0 and time.perf_counter() > deadline:
                    break
            if i == n:
                if self._misses:
                    with self._lock:
                        self._misses = 0
                return words[:n]
            with self._lock:
                self._misses += 1
                if self._misses >= self.MISSES_TO_SWITCH_OFF:
                    self._polling = False
        if isinstance(stream, torch.device):
            stream = torch.cuda.current_stream(stream)
        stream.synchronize()
        return words[:n]


_pinned_counts = _PinnedCounts()

# a float32 token row handed back as a view keeps its whole block alive; beyond this size the row is copied out instead
_DECODE_VIEW_MAX_WORDS = 1 << 17
_DECODE_WORKSPACE_WORDS = {}


def _on_device(dev):
    """Context that makes ``dev`` the current device; free when it already is."""
    return contextlib.nullcontext() if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)


def _viterbi_decode_call(name, B, L, ml, dev, extra_words, call):
    """Shared tail of the Viterbi decode calls: one allocation (workspace | tokens [B,L] int64 | predicted lengths [B] |
    tokens [B,L] float32 | ``extra_words`` more int64 words for the caller), the native call, the one wait, the emitted
    counts.  ``call`` receives (lib, stream handle, base address of the block, workspace words, address of the float32
    tokens, address of the pinned counts, address of the caller's words) and returns the status.  The kernels write the
    float32 tokens themselves, so nothing is enqueued behind the native call, and everything the host can do without the
    counts (the views of the results) it does while the kernels run."""
    lib = _lib.load()
    nodes = B * L
    fwords = (nodes + 1) // 2
    nwork = _DECODE_WORKSPACE_WORDS.get((B, L, ml))
    if nwork is None:
        nwork = _DECODE_WORKSPACE_WORDS[(B, L, ml)] = (lib.pcfgnat_viterbi_decode_workspace_bytes(B, L, ml) + 7) // 8
    with _on_device(dev):
        stream = torch.cuda.current_stream(dev)
        block = torch.empty((nwork + nodes + B + fwords + extra_words,), dtype=torch.int64, device=dev)
        base = block.data_ptr()
        # the emitted counts go straight into pinned host memory, which the device addresses like its own: the one
        # synchronisation of the decode is a wait for them (or for the stream), with no copy in front of it
        host = _pinned_counts.take(B)
        try:
            armed = _pinned_counts.arm(host, B, stream)
            rc = call(lib, stream.cuda_stream, base, nwork, base + 8 * (nwork + nodes + B), host.ptr,
                      base + 8 * (nwork + nodes + B + fwords))
            if rc != _lib.OK:
                _lib.check(rc, lib)
            pred = block[nwork + nodes:nwork + nodes + B]
            tokf = block[nwork + nodes + B:nwork + nodes + B + fwords].view(torch.float32)[:nodes].view(B, L)
            counts = _pinned_counts.wait(host, B, stream, armed)
        finally:
            _pinned_counts.give_back(host)
    return _emitted(tokf, counts, B, block), pred, block


def _emitted(tokf, counts, B, block):
    """The emitted part of the float32 token rows [B,L]: one sentence is a contiguous view of its row, the rows of a batch
    are copied together."""
    if B and min(counts) < 0:
        raise RuntimeError("viterbi_decoding: malformed traces")
    maxlen = max(counts) if B else 0
    tokens = tokf[:, :maxlen]
    if B != 1 or block.numel() > _DECODE_VIEW_MAX_WORDS:
        tokens = tokens.clone(memory_format=torch.contiguous_format)
    return tokens


def _viterbi_decode_ext(ext, logits, node_scores, node_tokens, links, output_length, left_tree_mask, pad_index, beta):
    """The decode calls through the torch extension: checks, allocation and enqueue in C++ (``viterbi_decode_enqueue``),
    the watch for the counts here.  Returns (tokens, pred_length, block, nodes)."""
    if links.dim() != 4:
        raise RuntimeError("pcfg_viterbi_decode: links must be float32 [bsz, prelen, max_left+1, prelen]")
    B, L = links.size(0), links.size(1)
    dev = links.device
    pen = _length_penalty(L // 4, beta, dev)
    host = _pinned_counts.take(B)
    try:
        tokf, pred, block, marked = ext.viterbi_decode_enqueue(logits, node_scores, node_tokens, links, output_length, left_tree_mask,
                                                               int(pad_index), pen, host.ptr, _pinned_counts.polling_on())
        counts = _pinned_counts.wait(host, B, dev, marked)
    finally:
        _pinned_counts.give_back(host)
    return _emitted(tokf, counts, B, block), pred, block, B * L


def _check_decode_graph(name, B, L, links, left_tree_mask):
    if links.dim() != 4 or links.dtype != torch.float32:
        raise RuntimeError("%s: links must be float32 [bsz, prelen, max_left+1, prelen]" % name)
    if links.size(0) != B or links.size(1) != L or links.size(3) != L:
        raise RuntimeError("%s: links shape %s does not match [bsz, prelen] = %s" % (name, tuple(links.shape), (B, L)))
    if left_tree_mask.dim() != 2 or left_tree_mask.size(0) != left_tree_mask.size(1):
        raise RuntimeError("%s: left_tree_mask must be square" % name)


def pcfg_viterbi_decode(unreduced_logits, links, output_length, unreduced_tokens, left_tree_mask, pad_index, beta=1.0):
    """The model's whole Viterbi decode (glat_decomposed_with_link_two_hands_tri_pcfg.py:483-502) in one native call:
    ``cuda_pcfg_viterbi`` -> length penalty ``arange ** beta`` -> NaN masking -> arg max over lengths >= 1 ->
    ``viterbi_decoding``.  Returns (tokens float32 [B, maxlen] right-padded with ``pad_index``, pred_length int64 [B]),
    the values the separate calls give."""
    ext = _ext()
    if ext is not None:
        tokens, pred, _, _ = _viterbi_decode_ext(ext, None, unreduced_logits, unreduced_tokens, links, output_length, left_tree_mask,
                                                 pad_index, beta)
        return tokens, pred
    _need_cuda("pcfg_viterbi_decode", unreduced_logits, links, output_length, unreduced_tokens, left_tree_mask)
    if unreduced_logits.dim() != 2 or links.dim() != 4:
        raise RuntimeError("pcfg_viterbi_decode: unreduced_logits must be [bsz, prelen] and links [bsz, prelen, max_left+1, prelen]")
    if unreduced_logits.dtype != torch.float32 or links.dtype != torch.float32:
        raise RuntimeError("pcfg_viterbi_decode: unreduced_logits and links must be float32")
    B, L = unreduced_logits.shape
    _check_decode_graph("pcfg_viterbi_decode", B, L, links, left_tree_mask)
    ml = links.size(2) - 1
    dev = unreduced_logits.device
    ob, links = unreduced_logits.contiguous(), links.contiguous()
    ol = _lengths("pcfg_viterbi_decode", output_length, B)
    tok = unreduced_tokens.to(dtype=torch.int64).contiguous()
    mask = left_tree_mask.to(dtype=torch.int64).contiguous()
    pen = _length_penalty(L // 4, beta, dev)

    def call(lib, stream, base, nwork, tokens_f32, counts, extra):
        return lib.pcfgnat_viterbi_decode(ob.data_ptr(), links.data_ptr(), ol.data_ptr(), tok.data_ptr(), mask.data_ptr(), mask.size(0),
                                          int(pad_index), pen.data_ptr(), base, base + 8 * nwork, tokens_f32, counts,
                                          base + 8 * (nwork + B * L), B, L, ml, stream)

    tokens, pred, _ = _viterbi_decode_call("pcfg_viterbi_decode", B, L, ml, dev, 0, call)
    return tokens, pred


def pcfg_viterbi_decode_logits(logits, links, output_length, left_tree_mask, pad_index, beta=1.0, return_nodes=False):
    """The decode as the model runs it, from the vocabulary logits [bsz, prelen, vocab] (float16 or float32):
    ``logits.log_softmax(-1).max(-1)`` (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416) and the Viterbi decode
    (:483-502) enqueued by one native call.  Returns what ``pcfg_viterbi_decode(*logsoftmax_max(logits), ...)`` returns:
    (tokens float32 [B, maxlen], pred_length int64 [B]); with ``return_nodes`` also the node scores [B,L] float32 and node
    tokens [B,L] int64 of the front-end."""
    ext = _ext()
    if ext is not None:
        tokens, pred, block, nodes = _viterbi_decode_ext(ext, logits, None, None, links, output_length, left_tree_mask, pad_index, beta)
        if not return_nodes:
            return tokens, pred
        tail = block[block.numel() - (nodes + (nodes + 1) // 2):]
        return tokens, pred, tail[nodes:].view(torch.float32)[:nodes].view(links.size(0), links.size(1)), \
            tail[:nodes].view(links.size(0), links.size(1))
    _need_cuda("pcfg_viterbi_decode_logits", logits, links, output_length, left_tree_mask)
    if logits.dim() != 3 or not logits.is_contiguous():
        raise RuntimeError("pcfg_viterbi_decode_logits: logits must be a contiguous [bsz, prelen, vocab] tensor")
    if logits.dtype not in (torch.float16, torch.float32):
        raise RuntimeError("pcfg_viterbi_decode_logits: logits must be float16 or float32 (got %s)" % logits.dtype)
    B, L, V = logits.shape
    _check_decode_graph("pcfg_viterbi_decode_logits", B, L, links, left_tree_mask)
    ml = links.size(2) - 1
    dev = logits.device
    links = links.contiguous()
    ol = _lengths("pcfg_viterbi_decode_logits", output_length, B)
    mask = left_tree_mask.to(dtype=torch.int64).contiguous()
    pen = _length_penalty(L // 4, beta, dev)
    code = _DTYPE_CODE[logits.dtype]
    nodes = B * L

    def call(lib, stream, base, nwork, tokens_f32, counts, idx):
        # the caller's words: node tokens [B,L] int64, then node scores [B,L] float32
        return lib.pcfgnat_viterbi_decode_logits(logits.data_ptr(), code, V, idx + 8 * nodes, idx, links.data_ptr(), ol.data_ptr(),
                                                 mask.data_ptr(), mask.size(0), int(pad_index), pen.data_ptr(), base, base + 8 * nwork,
                                                 tokens_f32, counts, base + 8 * (nwork + nodes), B, L, ml, stream)

    tokens, pred, block = _viterbi_decode_call("pcfg_viterbi_decode_logits", B, L, ml, dev, nodes + (nodes + 1) // 2, call)
    if not return_nodes:
        return tokens, pred
    tail = block[block.numel() - (nodes + (nodes + 1) // 2):]
    return tokens, pred, tail[nodes:].view(torch.float32)[:nodes].view(B, L), tail[:nodes].view(B, L)


def pcfg_lookahead_decode(links, unreduced_logits, unreduced_tokens, output_length, left_tree_mask, pad_index, beta=1.0,
                          strategy="lookahead", return_pointers=False):
    """The `lookahead` / `greedy` decode strategies (glat_decomposed_with_link_two_hands_tri_pcfg.py:419-481) in one
    launch: arg max pointers per node and the in-order walk.  Returns int64 tokens [B, maxlen] right-padded with
    ``pad_index`` (and the pointers ``k * prelen + c`` [B, prelen] if asked)."""
    if strategy not in ("lookahead", "greedy"):
        raise RuntimeError("pcfg_lookahead_decode: strategy must be 'lookahead' or 'greedy'")
    lib = get_pcfg_kernel()
    _need_cuda("pcfg_lookahead_decode", links, unreduced_tokens, output_length, left_tree_mask)
    if links.dim() != 4 or links.dtype != torch.float32 or links.size(1) != links.size(3):
        raise RuntimeError("pcfg_lookahead_decode: links must be float32 [bsz, prelen, max_left+1, prelen]")
    B, L, K, _ = links.shape
    dev = links.device
    links = links.contiguous()
    ob_ptr = None
    if strategy == "lookahead":
        _need_cuda("pcfg_lookahead_decode", unreduced_logits)
        if unreduced_logits.shape != (B, L) or unreduced_logits.dtype != torch.float32:
            raise RuntimeError("pcfg_lookahead_decode: unreduced_logits must be float32 [bsz, prelen]")
        ob = unreduced_logits.contiguous()
        ob_ptr = ob.data_ptr()
    if left_tree_mask.dim() != 2 or left_tree_mask.size(0) != left_tree_mask.size(1):
        raise RuntimeError("pcfg_lookahead_decode: left_tree_mask must be square")
    ol = _lengths("pcfg_lookahead_decode", output_length, B)
    tok = unreduced_tokens.to(dtype=torch.int64).contiguous()
    mask = left_tree_mask.to(dtype=torch.int64).contiguous()
    with torch.cuda.device(dev):
        idx = torch.empty((B, L), dtype=torch.int64, device=dev)
        out = torch.empty((B, L), dtype=torch.int64, device=dev)
        cnt = _pinned_counts.take(B)  # written by the kernel, read after the one stream wait
        try:
            armed = _pinned_counts.arm(cnt, B, torch.cuda.current_stream(dev))
            _lib.check(lib.pcfgnat_lookahead_decode(links.data_ptr(), ob_ptr, float(beta), ol.data_ptr(), tok.data_ptr(),
                                                    mask.data_ptr(), mask.size(0), int(pad_index), idx.data_ptr(), out.data_ptr(),
                                                    cnt.data_ptr(), B, L, K - 1, _stream(links)), lib)
            counts = _pinned_counts.wait(cnt, B, torch.cuda.current_stream(dev), armed)
        finally:
            _pinned_counts.give_back(cnt)
    if B and min(counts) < 0:
        raise RuntimeError("pcfg_lookahead_decode: the walk does not terminate")
    maxlen = max(counts) if B else 0
    tokens = out[:, :maxlen]
    return (tokens, idx) if return_pointers else tokens


def _criterion_args(name, logits, targets, links, output_length, target_length, matchmask, keep_word_mask):
    """Checks shared by the criterion entry points; returns (code, B, L, V, T, ml, Mc, targets, links, ol, tl, mask tensors)."""
    _need_cuda(name, logits, targets, links, output_length, target_length)
    if logits.dim() != 3 or not logits.is_contiguous():
        raise RuntimeError("%s: logits must be a contiguous [bsz, prelen, vocab] tensor" % name)
    B, L, V = logits.shape
    if targets.dim() != 2 or targets.size(0) != B or targets.dtype != torch.int64:
        raise RuntimeError("%s: targets must be an int64 [bsz, tarlen] tensor" % name)
    T = targets.size(1)
    code = _DTYPE_CODE.get(logits.dtype)
    if code is None or code == _lib.F64:
        raise RuntimeError("%s: logits must be float16 or float32" % name)
    if links.dim() != 4 or links.size(0) != B or links.size(1) != L or links.size(3) != L or links.dtype != torch.float32:
        raise RuntimeError("%s: links must be float32 [bsz, prelen, max_left+1, prelen]" % name)
    ml = links.size(2) - 1
    targets, links = targets.contiguous(), links.contiguous()
    ol = _lengths(name, output_length, B)
    tl = _lengths(name, target_length, B)
    Mc = (L - 2) // (ml + 1) + 1
    if (matchmask is None) != (keep_word_mask is None):
        raise RuntimeError("%s: matchmask and keep_word_mask go together" % name)
    mm8 = keep8 = None
    if matchmask is not None:
        _need_cuda(name, logits, matchmask, keep_word_mask)
        if tuple(matchmask.shape) != (B, T, L) or tuple(keep_word_mask.shape) != (B, L):
            raise RuntimeError("%s: matchmask must be [bsz, tarlen, prelen] and keep_word_mask [bsz, prelen]" % name)
        mm8 = matchmask.to(torch.uint8).contiguous()
        keep8 = keep_word_mask.to(torch.uint8).contiguous()
    return code, B, L, V, T, ml, Mc, targets, links, ol, tl, mm8, keep8


def pcfg_criterion_step(logits, targets, links, output_length, target_length, events=None, matchmask=None,
                        keep_word_mask=None, loss_scale=1.0):
    """The criterion's whole training pass in one native call (``pcfgnat_criterion_step``): ``logits`` [B,L,V] (fp16 or
    fp32, contiguous) is consumed in place and holds d loss / d logits afterwards.  ``events``: optional list of six
    ``torch.cuda.Event(enable_timing=True)`` (each recorded at least once before; entries may be None) that the library records before/after
    the gather forward, the inside forward + backward and the gather backward.
    ``matchmask`` [B,T,L] / ``keep_word_mask`` [B,L] (bool, as the glancing step returns them): the criterion's
    force-emit masking (nat_pcfg_loss.py:116-121); both None = off (``--no-force-emit``).  The rows of the pad nodes at
    or beyond a sentence's ``output_length`` feed nothing (neither sweep reads them, their gradient is zero): the gather
    forward leaves them unread (zeros in the returned ``match_all``) and the backward zeroes them without reading.
    ``loss_scale``: the factor the caller's loss carries downstream of the criterion (``loss * factor``,
    nat_pcfg_loss.py:139-140, times the fp16 loss scale) - a Python number, or a one-element float32 tensor on the device
    (no host read); both gradients come out multiplied by it, the factor entering in float32 ahead of the single rounding
    of d loss / d logits to the logits' dtype (pcfg_loss.py:77-83, 176-177).  The returned loss stays unscaled.  Returns
    (loss_and_invalid [2] float32, links_grad, ll [B], match_all_eos_masked, match_all_grad)."""
    lib = get_pcfg_kernel()
    code, B, L, V, T, ml, Mc, targets, links, ol, tl, mm8, keep8 = _criterion_args(
        "pcfg_criterion_step", logits, targets, links, output_length, target_length, matchmask, keep_word_mask)
    dev = logits.device
    mm_ptr = mm8.data_ptr() if mm8 is not None else None
    keep_ptr = keep8.data_ptr() if keep8 is not None else None
    scale_host, scale_dev = 1.0, None
    if torch.is_tensor(loss_scale):
        _need_cuda("pcfg_criterion_step", logits, loss_scale)
        if loss_scale.numel() != 1:
            raise RuntimeError("pcfg_criterion_step: loss_scale must be a number or a one-element tensor")
        scale_dev = loss_scale.detach().reshape(1).to(torch.float32)
    else:
        scale_host = float(loss_scale)
    ev_arr = None
    if events is not None:
        import ctypes
        if len(events) != 6:
            raise RuntimeError("pcfg_criterion_step: events must hold six torch.cuda.Event objects")
        ev_arr = (ctypes.c_void_p * 6)(*[(e.cuda_event if e is not None else None) for e in events])
    with torch.cuda.device(dev):
        match = torch.empty((B, L, T), dtype=torch.float32, device=dev)
        S = torch.empty((B, Mc, T + 2), dtype=torch.float32, device=dev)
        aux = torch.empty((max(1, lib.pcfgnat_pcfg_aux_floats(B, L, T, ml)),), dtype=torch.float32, device=dev)
        mg = torch.empty_like(match)
        lg = torch.empty_like(links)
        row_lse = torch.empty((B, L), dtype=torch.float32, device=dev)
        out = torch.empty((2,), dtype=torch.float32, device=dev)
        _lib.check(lib.pcfgnat_criterion_step(logits.data_ptr(), code, targets.data_ptr(), links.data_ptr(), ol.data_ptr(),
                                              tl.data_ptr(), mm_ptr, keep_ptr, match.data_ptr(), S.data_ptr(), aux.data_ptr(), mg.data_ptr(),
                                              lg.data_ptr(), row_lse.data_ptr(), out.data_ptr(), B, L, V, T, ml,
                                              scale_host, scale_dev.data_ptr() if scale_dev is not None else None,
                                              _stream(logits), ev_arr), lib)
    return out, lg, S[:, 0, 0], match, mg


def _criterion_forward(logits, targets, links, output_length, target_length, matchmask=None, keep_word_mask=None):
    """Forward half of the criterion pass (``pcfgnat_criterion_forward``): everything that does not depend on the loss's
    upstream gradient.  Returns (loss_and_invalid [2 + B], ll [B] with the invalid sentences zeroed, state) where ``state`` carries what
    ``_criterion_backward`` needs; ``logits`` must stay untouched until then (rows of pad nodes may already be zeroed)."""
    import ctypes
    lib = get_pcfg_kernel()
    code, B, L, V, T, ml, Mc, targets, links, ol, tl, mm8, keep8 = _criterion_args(
        "pcfg_criterion", logits, targets, links, output_length, target_length, matchmask, keep_word_mask)
    dev = logits.device
    pad_zeroed = ctypes.c_int(0)
    with torch.cuda.device(dev):
        match = torch.empty((B, L, T), dtype=torch.float32, device=dev)
        S = torch.empty((B, Mc, T + 2), dtype=torch.float32, device=dev)
        aux = torch.empty((max(1, lib.pcfgnat_pcfg_aux_floats(B, L, T, ml)),), dtype=torch.float32, device=dev)
        mg = torch.empty_like(match)
        lg = torch.empty_like(links)
        row_lse = torch.empty((B, L), dtype=torch.float32, device=dev)
        out = torch.empty((2 + B,), dtype=torch.float32, device=dev)  # loss, invalid count, ll with the invalid ones zeroed
        _lib.check(lib.pcfgnat_criterion_forward(logits.data_ptr(), code, targets.data_ptr(), links.data_ptr(), ol.data_ptr(),
                                                 tl.data_ptr(), mm8.data_ptr() if mm8 is not None else None,
                                                 keep8.data_ptr() if keep8 is not None else None, match.data_ptr(), S.data_ptr(),
                                                 aux.data_ptr(), mg.data_ptr(), lg.data_ptr(), row_lse.data_ptr(), out.data_ptr(),
                                                 out.data_ptr() + 8, ctypes.byref(pad_zeroed), B, L, V, T, ml, _stream(logits)), lib)
    state = {"targets": targets, "match_all_grad": mg, "links_grad": lg, "row_lse": row_lse, "keep": keep8, "output_length": ol,
             "pad_rows_zeroed": int(pad_zeroed.value), "dims": (code, B, L, V, T, ml)}
    return out, out[2:], state


def _criterion_backward(logits, state, upstream):
    """Backward half (``pcfgnat_criterion_backward``): ``logits`` becomes ``upstream`` * d loss / d logits in place and the
    saved rule gradients are multiplied by ``upstream`` (a one-element tensor on the device; it is never read by the
    host).  Returns (logits, links_grad)."""
    lib = get_pcfg_kernel()
    code, B, L, V, T, ml = state["dims"]
    up = upstream.detach().reshape(1).to(device=logits.device, dtype=torch.float32)
    keep8 = state["keep"]
    with torch.cuda.device(logits.device):
        _lib.check(lib.pcfgnat_criterion_backward(logits.data_ptr(), code, state["targets"].data_ptr(), state["match_all_grad"].data_ptr(),
                                                  state["row_lse"].data_ptr(), keep8.data_ptr() if keep8 is not None else None,
                                                  state["output_length"].data_ptr(), state["pad_rows_zeroed"], up.data_ptr(),
                                                  state["links_grad"].data_ptr(), B, L, V, T, ml, _stream(logits)), lib)
    return logits, state["links_grad"]


class PCFGCriterionFunc(Function):
    """The criterion's loss (nat_pcfg_loss.py:98-145) as one differentiable op.  Like the reference's own ops
    (pcfg_loss.py:67-73 runs the inside backward eagerly inside the forward; :144-181 hands the logits buffer back as the
    gradient) the forward does everything that does not depend on the upstream gradient of the loss - gather, both inside
    sweeps, the posteriors at an upstream gradient of 1, the loss - and returns the logits buffer marked dirty (it must not
    be used any more).  The backward is one native call: a single read + write pass turns the logits into their gradient,
    with the upstream gradient (e.g. the fp16 loss scale) folded in on the device, in float32, ahead of the one rounding
    to the logits' dtype, as pcfg_loss.py:77-83 and :176-177 do; nothing is read back by the host.  May run backward once."""

    @staticmethod
    def forward(ctx, outputs, links, targets, output_length, target_length, matchmask, keep_word_mask):
        need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        if need:
            out, ll, state = _criterion_forward(outputs, targets, links, output_length, target_length, matchmask, keep_word_mask)
            ctx.state = state
            ctx.save_for_backward(outputs)
            ctx.has_backward = False
        else:  # nothing to differentiate: the plain step (its gradients are discarded)
            out, _, ll, _, _ = pcfg_criterion_step(outputs, targets, links, output_length, target_length, matchmask=matchmask,
                                                   keep_word_mask=keep_word_mask)
            ll = ll.masked_fill(ll.isinf().logical_or(ll.isnan()), 0)
        ctx.mark_dirty(outputs)
        ctx.set_materialize_grads(False)
        return outputs, out[0], ll, out[1]

    @staticmethod
    def backward(ctx, grad_outputs, grad_loss, grad_ll, grad_invalid):
        assert grad_outputs is None, "Cannot reuse the logits after pcfg_criterion"
        assert grad_ll is None, "pcfg_criterion: only the loss is differentiable (use cuda_pcfg_loss for per-sentence gradients)"
        if grad_loss is None:
            return (None,) * 7
        assert not ctx.has_backward, "Cannot backward twice in pcfg_criterion"
        ctx.has_backward = True
        (buf,) = ctx.saved_tensors
        buf, links_grad = _criterion_backward(buf, ctx.state, grad_loss)
        ctx.state = None
        return (buf if ctx.needs_input_grad[0] else None, links_grad if ctx.needs_input_grad[1] else None, None, None, None, None,
                None)


def pcfg_criterion(outputs, targets, links, output_length, target_length, matchmask=None, keep_word_mask=None):
    """loss = -(log-likelihood / target_length).mean() over the sentences with a finite log-likelihood, differentiable in
    ``outputs`` [B,L,V] (fp16/fp32 logits, consumed in place) and ``links``; one native call in the forward, one in the
    backward.  Returns
    (loss, ll [B] with invalid sentences zeroed, number of invalid sentences) - the dict entries of
    ``harness.compute_pcfg_loss``."""
    ext = _ext()
    if ext is not None and outputs.is_cuda:
        return ext.pcfg_criterion(outputs, targets, links, output_length, target_length, matchmask, keep_word_mask)
    _, loss, ll, invalid = PCFGCriterionFunc.apply(outputs, links, targets, output_length, target_length, matchmask, keep_word_mask)
    return loss, ll, invalid

