"""TEST INFRASTRUCTURE ONLY: numpy/ctypes front-end of the CPU oracle (oracle/pcfg_oracle.c).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this
module.  The product package never does: it talks to the HIP library and fails loudly without it.

Each function mirrors one entry of the reference's native module (fs_plugins/custom_ops/pcfg_loss.cpp:76-81)
on numpy arrays; ``dtype`` selects the float32 or float64 instantiation of the C loops.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_c_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    so = os.path.join(_HERE, "liboracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return so


def _lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        _LIB = ctypes.CDLL(so)
        _LIB.oracle_num_threads.restype = ctypes.c_int
    return _LIB


def num_threads():
    return int(_lib().oracle_num_threads())


def set_num_threads(n):
    _lib().oracle_set_num_threads(int(n))


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "_f32", ctypes.c_float
    if dtype == np.float64:
        return "_f64", ctypes.c_double
    raise TypeError("oracle computes in float32 or float64, got %s" % dtype)


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def table_sizes(L, ml):
    """(Mc, Lc) = main-chain and local-tree table heights (pcfg_loss.cu:389-390)."""
    Mc = (L - 2) // (ml + 1) + 1
    return Mc, L - Mc


def lsg_fwd(x, idx, want_probs=False, dtype=np.float64):
    """logsoftmax_gather (logsoftmax_gather.cu:295-359).  x: [B,L,V] any float dtype, idx: [B,L,T] int64 with
    arbitrary strides (the criterion passes a stride-0 expanded view).  Returns (sel [B,L,T], probs [B,L,V] | None),
    both in ``dtype``; rounding ``probs`` to the logits dtype is the caller's business."""
    sfx, _ = _sfx(dtype)
    B, L, V = x.shape
    T = idx.shape[2]
    xw = _c(x.reshape(B * L, V), dtype)
    assert idx.dtype == np.int64 and idx.shape[:2] == (B, L)
    item = idx.itemsize
    s0, s1, s2 = (s // item for s in idx.strides)
    # Address arithmetic relative to the first element of the view, rows enumerated as b*L+p.
    base = (np.arange(B, dtype=np.int64)[:, None] * s0 + np.arange(L, dtype=np.int64)[None, :] * s1).reshape(-1)
    base = np.ascontiguousarray(base)
    sel = np.empty((B * L, T), dtype=dtype)
    probs = np.empty((B * L, V), dtype=dtype) if want_probs else None
    idx_ptr = ctypes.c_void_p(idx.ctypes.data)
    getattr(_lib(), "oracle_lsg_fwd" + sfx)(
        _p(xw), idx_ptr, _p(base), ctypes.c_int64(s2), _p(sel), _p(probs) if want_probs else None,
        ctypes.c_int64(B * L), ctypes.c_int64(V), ctypes.c_int64(T))
    return sel.reshape(B, L, T), (probs.reshape(B, L, V) if want_probs else None)


def lsg_bwd(probs, idx, grad_sel, dtype=np.float64):
    """Backward of logsoftmax_gather as DagLogsoftmaxGatherFunc.backward performs it (pcfg_loss.py:176-177), without the
    rounding to the buffer dtype.  Returns the gradient w.r.t. the logits [B,L,V] in ``dtype``."""
    sfx, _ = _sfx(dtype)
    B, L, V = probs.shape
    T = idx.shape[2]
    buf = np.array(probs.reshape(B * L, V), dtype=dtype, order="C", copy=True)
    g = _c(grad_sel.reshape(B * L, T), dtype)
    item = idx.itemsize
    s0, s1, s2 = (s // item for s in idx.strides)
    base = np.ascontiguousarray(
        (np.arange(B, dtype=np.int64)[:, None] * s0 + np.arange(L, dtype=np.int64)[None, :] * s1).reshape(-1))
    getattr(_lib(), "oracle_lsg_bwd" + sfx)(_p(buf), ctypes.c_void_p(idx.ctypes.data), _p(base), ctypes.c_int64(s2), _p(g),
                                             ctypes.c_int64(B * L), ctypes.c_int64(V), ctypes.c_int64(T))
    return buf.reshape(B, L, V)


def inside_fwd(match, links, out_len, tgt_len, dtype=np.float64):
    """pcfg_loss (pcfg_loss.cu:379-401).  Returns (S [B,Mc,T+2], C [B,Lc,T+2,ml+2]); ll = S[:,0,0]."""
    sfx, _ = _sfx(dtype)
    B, L, T = match.shape
    ml = links.shape[2] - 1
    assert links.shape == (B, L, ml + 1, L)
    Mc, Lc = table_sizes(L, ml)
    match, links = _c(match, dtype), _c(links, dtype)
    out_len, tgt_len = _c(out_len, np.int64), _c(tgt_len, np.int64)
    S = np.empty((B, Mc, T + 2), dtype=dtype)
    C = np.empty((B, Lc, T + 2, ml + 2), dtype=dtype)
    getattr(_lib(), "oracle_inside_fwd" + sfx)(_p(match), _p(links), _p(out_len), _p(tgt_len), _p(S), _p(C),
                                                B, L, T, ml)
    return S, C


def inside_bwd(grad_out, S, C, match, links, out_len, tgt_len, dtype=np.float64):
    """pcfg_loss_backward (pcfg_loss_backward.cu:654-721), exact-gradient reading.
    Returns (match_grad [B,L,T], links_grad [B,L,ml+1,L])."""
    sfx, _ = _sfx(dtype)
    B, L, T = match.shape
    ml = links.shape[2] - 1
    match, links, S, C = _c(match, dtype), _c(links, dtype), _c(S, dtype), _c(C, dtype)
    grad_out = _c(grad_out, dtype)
    out_len, tgt_len = _c(out_len, np.int64), _c(tgt_len, np.int64)
    Sg, Cg = np.empty_like(S), np.empty_like(C)
    mg, lg = np.empty_like(match), np.empty_like(links)
    getattr(_lib(), "oracle_inside_bwd" + sfx)(_p(grad_out), _p(S), _p(C), _p(match), _p(links), _p(out_len),
                                                _p(tgt_len), _p(Sg), _p(Cg), _p(mg), _p(lg), B, L, T, ml)
    return mg, lg


def best_tree(S, C, match, links, out_len, tgt_len, dtype=np.float64, return_margin=False):
    """pcfg_best_tree (pcfg_best_tree.cu:333-360) on given inside tables.  Returns tree [B,L] int64; with
    ``return_margin`` also a [B,3] array about the arg-max decisions of the trace: the smallest gap between the best and
    the second-best candidate (0 = an exact tie, inf = no decision had two finite candidates), the number of exact ties,
    the smallest gap that is not a tie."""
    sfx, _ = _sfx(dtype)
    B, L, T = match.shape
    ml = links.shape[2] - 1
    match, links, S, C = _c(match, dtype), _c(links, dtype), _c(S, dtype), _c(C, dtype)
    out_len, tgt_len = _c(out_len, np.int64), _c(tgt_len, np.int64)
    tree = np.empty((B, L), dtype=np.int64)
    margin = np.empty((B, 3), dtype=dtype) if return_margin else None
    getattr(_lib(), "oracle_best_tree" + sfx)(_p(S), _p(C), _p(match), _p(links), _p(out_len), _p(tgt_len), _p(tree),
                                               _p(margin) if return_margin else None, B, L, T, ml)
    return (tree, margin) if return_margin else tree


def viterbi(ob, links, out_len, dtype=np.float32, return_margin=False):
    """pcfg_viterbi (pcfg_viterbi.cu:272-301).  Returns (S [B,L,L//4], R, Lt, M [B,L,L//4] int64); the autograd
    wrapper exposes scores = S[:,1,:] (pcfg_loss.py:136).  With ``return_margin`` a fifth value: the [B,3] margin
    array of ``best_tree``, over all table entries."""
    sfx, _ = _sfx(dtype)
    B, L = ob.shape
    ml = links.shape[2] - 1
    Lq = L // 4
    ob, links = _c(ob, dtype), _c(links, dtype)
    out_len = _c(out_len, np.int64)
    S = np.empty((B, L, Lq), dtype=dtype)
    Cv = np.empty((B, L, Lq), dtype=dtype)
    R = np.empty((B, L, Lq), dtype=np.int64)
    Lt = np.empty((B, L, Lq), dtype=np.int64)
    M = np.empty((B, L, Lq), dtype=np.int64)
    margin = np.empty((B, 3), dtype=dtype) if return_margin else None
    getattr(_lib(), "oracle_viterbi" + sfx)(_p(ob), _p(links), _p(out_len), _p(S), _p(Cv), _p(R), _p(Lt), _p(M),
                                             _p(margin) if return_margin else None, B, L, ml)
    return (S, R, Lt, M, margin) if return_margin else (S, R, Lt, M)


def viterbi_decoding(pred_length, output_length, L_trace, R_trace, M_trace, unreduced_tokens, left_tree_mask, pad_index):
    """viterbi_decoding (pcfg_loss.cpp:12-73).  Returns float32 [B, maxlen] right-padded with pad_index
    (the reference can only assemble equal-length rows, :68; ragged batches get the evidently intended padding)."""
    B, L, Lq = L_trace.shape
    pred_length, output_length = _c(pred_length, np.int64), _c(output_length, np.int64)
    Lt, R, M = _c(L_trace, np.int64), _c(R_trace, np.int64), _c(M_trace, np.int64)
    tokens, mask = _c(unreduced_tokens, np.int64), _c(left_tree_mask, np.int64)
    cap = L
    out = np.full((B, cap), pad_index, dtype=np.int64)
    out_len = np.zeros(B, dtype=np.int64)
    _lib().oracle_viterbi_decoding(_p(pred_length), _p(output_length), _p(Lt), _p(R), _p(M), _p(tokens), _p(mask),
                                   ctypes.c_int64(mask.shape[0]), ctypes.c_int64(pad_index), _p(out), _p(out_len),
                                   B, L, Lq, cap)
    if (out_len < 0).any():
        raise RuntimeError("viterbi_decoding: malformed traces")
    maxlen = int(out_len.max()) if B else 0
    return out[:, :maxlen].astype(np.float32)


def lookahead_decode(links, unreduced_logits, output_length, unreduced_tokens, left_tree_mask, pad_index, beta=1.0):
    """`lookahead` decode (glat_decomposed_with_link_two_hands_tri_pcfg.py:419-481); ``unreduced_logits=None`` gives the
    `greedy` strategy (:432-434).  Returns (tokens int64 [B, maxlen] right-padded with pad_index, links_idx [B, L])."""
    links = _c(links, np.float32)
    B, L, K, _ = links.shape
    ob = None if unreduced_logits is None else _c(unreduced_logits, np.float32)
    output_length = _c(output_length, np.int64)
    tokens, mask = _c(unreduced_tokens, np.int64), _c(left_tree_mask, np.int64)
    cap = L
    idx = np.zeros((B, L), dtype=np.int64)
    out = np.full((B, cap), pad_index, dtype=np.int64)
    out_len = np.zeros(B, dtype=np.int64)
    _lib().oracle_lookahead_decode(_p(links), _p(ob) if ob is not None else None, ctypes.c_float(beta), _p(output_length),
                                   _p(tokens), _p(mask), ctypes.c_int64(mask.shape[0]), ctypes.c_int64(pad_index), _p(idx),
                                   _p(out), _p(out_len), B, L, K - 1, cap)
    if (out_len < 0).any():
        raise RuntimeError("lookahead_decode: the walk does not terminate")
    maxlen = int(out_len.max()) if B else 0
    return out[:, :maxlen], idx
