"""GPU parity tests: the HIP path (through the operator API, which calls the C-ABI) against the CPU oracle and torch's
library routines on identical seeded inputs.

Bars: integer outputs (trees, traces, decoded tokens) bit-exact; viterbi scores bit-exact (same fp32 association
order); fp32 log-likelihoods within 1e-5 relative, gradients within 1e-4 of the gradient scale; fp16 buffers within
one fp16 rounding step.
"""
import math

import numpy as np
import pytest

import gradcheck
import torch

from oracle import oracle
from pcfg_nat_amd import custom_ops as ops
from pcfg_nat_amd import harness, synth

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _gather_ref(x, idx):
    return torch.log_softmax(x.float() if x.dtype != torch.float64 else x, -1).gather(-1, idx)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("V", [7, 512, 1001, 40000, 50257])
def test_lsg_forward_and_inplace_softmax(dtype, V):
    g = torch.Generator().manual_seed(V)
    B, L, T = 3, 5, 9
    x = (torch.randn(B, L, V, generator=g) * 2).to(dtype)
    tgt = torch.randint(0, V, (B, T), generator=g)
    idx = tgt.unsqueeze(1).expand(-1, L, -1)
    xd = x.to(DEV)
    keep = xd.clone()
    # no gradient: logits untouched
    sel = ops._logsoftmax_gather(xd, idx.to(DEV), False)
    assert torch.equal(xd, keep)
    want = _gather_ref(x, idx)
    tol = 1e-12 if dtype == torch.float64 else 2e-5
    assert sel.dtype == (torch.float64 if dtype == torch.float64 else torch.float32)
    assert torch.allclose(sel.cpu(), want, rtol=tol, atol=tol)
    # oracle agrees too (rows enumerated by the C loops)
    osel, oprobs = oracle.lsg_fwd(x.numpy(), idx.numpy(), want_probs=True)
    assert np.allclose(sel.cpu().numpy(), osel, rtol=tol, atol=tol)
    # with gradient: same gathered values, logits replaced by softmax in their own dtype
    sel2 = ops._logsoftmax_gather(xd, idx.to(DEV), True)
    assert torch.allclose(sel2, sel, rtol=tol, atol=tol)
    probs = torch.from_numpy(oprobs)
    got = xd.cpu().double()
    if dtype == torch.float16:
        assert (got - probs).abs().max() <= (probs.abs() * 2 ** -10 + 2 ** -24).max()
        assert torch.allclose(got, probs, rtol=2 ** -10, atol=2 ** -24)
    elif dtype == torch.float32:
        assert torch.allclose(got, probs, rtol=1e-5, atol=1e-10)
    else:
        assert torch.allclose(got, probs, rtol=1e-12, atol=1e-300)


def test_lsg_misaligned_rows_and_strided_indices():
    """V odd => rows start at every 2-byte alignment; index tensor genuinely 3-d and non-contiguous."""
    g = torch.Generator().manual_seed(5)
    B, L, V, T = 2, 9, 333, 6
    x = (torch.randn(B, L, V, generator=g) * 3).half()
    idx = torch.randint(0, V, (B, T, L), generator=g).transpose(1, 2)
    xd = x.to(DEV)
    sel = ops._logsoftmax_gather(xd, idx.to(DEV), True)
    assert torch.allclose(sel.cpu(), _gather_ref(x, idx), rtol=2e-5, atol=2e-5)
    want_p = torch.softmax(x.float(), -1)
    assert torch.allclose(xd.cpu().float(), want_p, rtol=2 ** -10, atol=2 ** -24)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_lsg_backward_matches_torch_ops(dtype):
    """The fused backward against the reference's own two torch calls (pcfg_loss.py:176-177) on the same buffer."""
    g = torch.Generator().manual_seed(9)
    B, L, V, T = 4, 6, 2048, 12
    probs = torch.softmax(torch.randn(B, L, V, generator=g) * 2, -1).to(dtype).to(DEV)
    tgt = torch.randint(0, V, (B, T), generator=g)
    tgt[:, 3] = tgt[:, 1]  # duplicate columns
    tgt[:, 7:] = 1         # pads
    idx = tgt.unsqueeze(1).expand(-1, L, -1).to(DEV)
    gout = torch.randn(B, L, T, generator=g).to(DEV)
    gout[:, :, 7:] = 0
    ref = probs.clone()
    ref.mul_(gout.sum(-1, keepdim=True).neg_().to(ref.dtype))
    ref.scatter_add_(-1, idx, gout.to(ref.dtype))
    got = probs.clone()
    ops._logsoftmax_gather_backward(got, idx, gout)
    if dtype == torch.float16:
        # the row factor -(sum g) is rounded to fp16 from differently ordered fp32 sums: allow one rounding step
        assert torch.allclose(got.float(), ref.float(), rtol=2 ** -9, atol=2 ** -20)
        same = (got == ref).float().mean().item()
        assert same > 0.99
    else:
        assert torch.allclose(got, ref, rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("dtype,V,T", [(torch.float16, 16384, 24), (torch.float32, 16384, 24), (torch.float32, 30001, 40),
                                       (torch.float16, 50000, 600)])
def test_lsg_backward_adds_duplicate_targets_in_target_order(dtype, V, T):
    """Targets that share a column are added one after the other in the order of the target positions (scatter_add_ along
    the last dimension, pcfg_loss.py:177), however they reach the thread that owns the column: three of one column (sorted
    on arrival), six of another (more than the thread keeps: it goes through all targets), columns of one thread's
    different chunks, two elements of one chunk.  The upstream gradients are multiples of 2^-5, so that their sum is exact
    in any order and every bit of the result is fixed: compared for equality with the same operations one at a time.
    The larger vocabularies have rows with more 16-byte chunks than a thread keeps in registers (targets in those chunks
    too, the odd one with rows that start off the 16-byte grid), the last case more than 512 targets per row."""
    g = torch.Generator().manual_seed(21)
    B, L = 2, 5
    epv = 8 if dtype == torch.float16 else 4
    probs = torch.softmax(torch.randn(B, L, V, generator=g) * 2, -1).to(dtype)
    tgt = torch.randint(0, V, (B, T), generator=g)
    a, b, c = 1000, 3001, 77
    tgt[:, [2, 9, 15]] = a
    tgt[:, [0, 4, 5, 11, 20, 23]] = b
    tgt[:, 6] = c
    tgt[:, 7] = c + 1                # the same 16-byte chunk
    tgt[:, 8] = c + 512 * epv        # the same thread's next chunk
    tgt[:, 10] = c + 2 * 512 * epv
    if V > 10 * 512 * epv + 100:     # chunks beyond the ten a thread keeps in registers: one target, a pair, a triple
        far = 10 * 512 * epv + 40
        tgt[:, 12] = far
        tgt[:, [13, 16]] = far + 3 * epv + 1
        tgt[:, [14, 17, 19]] = V - 2
    idx = tgt.unsqueeze(1).expand(-1, L, -1).contiguous()
    gout = torch.randint(-40, 41, (B, L, T), generator=g).float() / 32
    # one rounding to the buffer's dtype per operation, the targets one after the other
    ref = probs.clone()
    ref.mul_(gout.sum(-1, keepdim=True).neg_().to(ref.dtype))
    for t in range(T):
        for b_ in range(B):
            col = int(tgt[b_, t])
            ref[b_, :, col] = (ref[b_, :, col].float() + gout[b_, :, t].to(dtype).float()).to(dtype)
    if dtype == torch.float32:  # which is what torch's own call does on the CPU
        ref2 = probs.clone()
        ref2.mul_(gout.sum(-1, keepdim=True).neg_())
        ref2.scatter_add_(-1, idx, gout)
        assert torch.equal(ref, ref2)
    got = probs.clone().to(DEV)
    ops._logsoftmax_gather_backward(got, idx.to(DEV), gout.to(DEV))
    assert torch.equal(got.cpu(), ref)
    # the recomputing backward (row log-sum-exps instead of probabilities in the buffer) adds in float32 and rounds once
    x = (torch.randn(B, L, V, generator=g) * 2).to(dtype)
    xd = x.to(DEV)
    sel, lse = ops._logsoftmax_gather_lse(xd, idx.to(DEV))
    ops._logsoftmax_gather_backward_lse(xd, idx.to(DEV), gout.to(DEV), lse)
    want = torch.exp(x.float() - lse.cpu().unsqueeze(-1)) * gout.sum(-1, keepdim=True).neg_()
    for t in range(T):
        for b_ in range(B):
            want[b_, :, int(tgt[b_, t])] += gout[b_, :, t]
    assert torch.allclose(xd.cpu().float(), want.to(dtype).float(), rtol=2 ** -9 if dtype == torch.float16 else 1e-5, atol=1e-7)
    at = torch.zeros(B, V, dtype=torch.bool)
    at.scatter_(1, tgt, True)
    cols = at.unsqueeze(1).expand(-1, L, -1)
    assert torch.allclose(xd.cpu().float()[cols], want[cols], rtol=2 ** -10 if dtype == torch.float16 else 2e-6, atol=1e-7)


@pytest.mark.parametrize("dtype,V", [(torch.float16, 2048), (torch.float16, 333), (torch.float32, 1001), (torch.float64, 257)])
def test_lsg_lse_split_matches_autograd(dtype, V):
    """Read-only forward + recomputing backward against torch's own log_softmax/gather gradient in float64."""
    g = torch.Generator().manual_seed(11)
    B, L, T = 3, 7, 12
    x = (torch.randn(B, L, V, generator=g) * 3).to(dtype)
    tgt = torch.randint(0, V, (B, T), generator=g)
    tgt[:, 3] = tgt[:, 1]  # duplicate columns
    tgt[:, 9:] = 1         # pads
    idx = tgt.unsqueeze(1).expand(-1, L, -1)
    gout = torch.randn(B, L, T, generator=g)
    gout[:, :, 9:] = 0
    ol = torch.tensor([7, 5, 6])
    tl = torch.tensor([9, 4, 6])
    xd = x.to(DEV)
    sel, lse = ops._logsoftmax_gather_lse(xd, idx.to(DEV), eos_lengths=(ol.to(DEV), tl.to(DEV)))
    assert torch.equal(xd.cpu(), x)  # forward leaves the logits alone
    leaf = x.double().requires_grad_(True)
    ref_sel = torch.log_softmax(leaf, -1).gather(-1, idx)
    ref_lse = torch.logsumexp(leaf.detach(), -1)
    want = harness.eos_masked(ref_sel.detach(), ol, tl)
    fin = torch.isfinite(want)
    tol = 1e-12 if dtype == torch.float64 else 2e-5
    assert torch.equal(torch.isfinite(sel.cpu()), fin)
    assert torch.allclose(sel.cpu().double()[fin], want[fin], rtol=tol, atol=tol)
    assert torch.allclose(lse.cpu().double(), ref_lse, rtol=tol, atol=tol)
    gdev = gout.to(DEV).to(sel.dtype)
    ops._logsoftmax_gather_backward_lse(xd, idx.to(DEV), gdev, lse)
    (ref_sel * gout.double()).sum().backward()
    got = xd.cpu().double()
    if dtype == torch.float16:
        # one rounding to fp16 of the float32 result
        assert torch.allclose(got, leaf.grad, rtol=2 ** -10, atol=2 ** -24)
    elif dtype == torch.float32:
        assert torch.allclose(got, leaf.grad, rtol=1e-5, atol=1e-7)
    else:
        assert torch.allclose(got, leaf.grad, rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize("dtype,V", [(torch.float16, 40000), (torch.float16, 333), (torch.float32, 1001), (torch.float64, 257),
                                     (torch.float16, 48000)])
def test_logsoftmax_max_matches_torch(dtype, V):
    g = torch.Generator().manual_seed(V)
    B, L = 2, 5
    x = (torch.randn(B, L, V, generator=g) * 3).to(dtype)
    x[0, 1, 7] = x[0, 1].max()   # exact ties: the first position wins
    x[0, 1, V - 3] = x[0, 1, 7]
    x[1, 2, :] = 0.5             # a constant row
    x[1, 3, 5:9] = -math.inf
    best, idx = ops.logsoftmax_max(x.to(DEV))
    want_best, want_idx = torch.log_softmax(x.double(), -1).max(-1)
    first = (x == x.max(-1, keepdim=True)[0]).int().argmax(-1)   # first maximum
    assert torch.equal(idx.cpu(), first)
    assert torch.equal(x.gather(-1, idx.cpu().unsqueeze(-1)), x.gather(-1, want_idx.unsqueeze(-1)))
    tol = 1e-12 if dtype == torch.float64 else 2e-6
    assert torch.allclose(best.cpu().double(), want_best, rtol=tol, atol=tol)


def test_lsg_autograd_contract():
    g = torch.Generator().manual_seed(2)
    B, L, V, T = 2, 4, 640, 5
    leaf = (torch.randn(B, L, V, generator=g)).to(DEV).requires_grad_(True)
    x = leaf * 1.0  # non-leaf, as in the model
    tgt = torch.randint(0, V, (B, T), generator=g).to(DEV)
    idx = tgt.unsqueeze(1).expand(-1, L, -1)
    out, sel = ops.dag_logsoftmax_gather_inplace(x, idx)
    assert out.data_ptr() == x.data_ptr()
    w = torch.randn(B, L, T, generator=g).to(DEV)
    (sel * w).sum().backward()
    ref_leaf = leaf.detach().clone().requires_grad_(True)
    (torch.log_softmax(ref_leaf, -1).gather(-1, idx) * w).sum().backward()
    assert torch.allclose(leaf.grad, ref_leaf.grad, rtol=1e-4, atol=1e-6)
    # no gradient requested: buffer untouched, no graph
    y = torch.randn(B, L, V, generator=g).to(DEV)
    keep = y.clone()
    out, sel = ops.dag_logsoftmax_gather_inplace(y, idx)
    assert torch.equal(y, keep) and not sel.requires_grad


def _oracle_inside(batch, match):
    links = batch["links"].numpy()
    ol, tl = batch["output_length"].numpy(), batch["target_length"].numpy()
    S, C = oracle.inside_fwd(match, links, ol, tl, dtype=np.float64)
    mg, lg = oracle.inside_bwd(np.ones(len(ol)), S, C, match, links, ol, tl, dtype=np.float64)
    return S, C, mg, lg


def _train_case(name):
    if name == "cfg1":
        return synth.config1()
    if name == "wmt_small":  # config-2 shaped, smaller vocabulary and batch
        return synth.config2(B=6, V=1000, seed=1, logit_dtype=torch.float32)
    if name == "ragged_short":
        return synth.training_batch(5, 64, 12, 300, [64, 40, 22, 8, 4], [12, 9, 7, 3, 2], seed=8)
    if name == "L128_T100":  # the longest targets the paired sweeps hold in LDS; one target too long for its graph
        return synth.training_batch(4, 128, 100, 60, [128, 100, 20, 6], [100, 64, 60, 3], seed=18)
    if name == "L126_T96":  # an odd number of main-chain nodes
        return synth.training_batch(3, 126, 96, 60, [126, 126, 70], [96, 2, 51], seed=19)
    if name == "L128_T104":  # just beyond: forward and outside sweeps as separate launches
        return synth.training_batch(2, 128, 104, 60, [128, 96], [104, 80], seed=20)
    if name == "L130":  # 65 main-chain nodes: the first shape of the pipelined sweeps
        return synth.training_batch(3, 130, 30, 100, [130, 128, 66], [30, 30, 17], seed=21)
    if name == "L132":
        return synth.training_batch(2, 132, 34, 100, [132, 130], [34, 29], seed=22)
    if name == "L1028":  # 514 main-chain nodes: the first shape beyond the pipelined sweeps
        return synth.training_batch(2, 1028, 16, 50, [1028, 1026], [16, 13], seed=23)
    if name == "L256":
        return synth.training_batch(3, 256, 40, 200, [256, 200, 130], [40, 33, 38], seed=12)
    if name == "L512":  # streaming kernels, emissions staged in LDS
        return synth.training_batch(3, 512, 30, 100, [512, 300, 258], [30, 25, 30], seed=13)
    if name == "L512_long":  # config-3 shaped: streaming kernels, emissions read from global memory
        return synth.training_batch(2, 512, 140, 100, [512, 444], [140, 120], seed=14)
    if name == "L320_mixed":  # pipelined sweeps: a full sentence, a target too long for its graph (-inf), a minimal one
        return synth.training_batch(3, 320, 40, 100, [320, 20, 4], [40, 30, 2], seed=16)
    if name == "L2050":  # beyond the pipelined sweeps: one workgroup per sentence streams the link rows
        return synth.training_batch(2, 2050, 6, 50, [2050, 1400], [6, 5], seed=17)
    if name == "L1026":
        return synth.training_batch(2, 1026, 20, 50, [1026, 600], [20, 17], seed=15)
    raise KeyError(name)


def _match_for(batch):
    sel = torch.log_softmax(batch["logits"].double(), -1).gather(
        -1, batch["targets"].unsqueeze(1).expand(-1, batch["logits"].shape[1], -1))
    return harness.eos_masked(sel.float(), batch["output_length"], batch["target_length"])


@pytest.mark.parametrize("case", ["cfg1", "wmt_small", "ragged_short", "L128_T100", "L126_T96", "L128_T104", "L130", "L132", "L256",
                                  "L320_mixed", "L512", "L512_long", "L1026", "L1028", "L2050"])
def test_inside_forward_backward_vs_oracle(case):
    batch = _train_case(case)
    match = _match_for(batch)
    S64, C64, mg64, lg64 = _oracle_inside(batch, match.numpy())
    md = match.to(DEV).requires_grad_(True)
    ld = batch["links"].to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, batch["output_length"].to(DEV), batch["target_length"].to(DEV))
    want_ll = S64[:, 0, 0]
    got_ll = ll.detach().cpu().double().numpy()
    fin = np.isfinite(want_ll)
    assert fin.any()
    assert np.array_equal(np.isfinite(got_ll), fin)
    assert np.allclose(got_ll[fin], want_ll[fin], rtol=1e-5)
    w = torch.linspace(0.5, 1.5, ll.numel(), device=DEV)
    (ll.masked_fill(~torch.isfinite(ll), 0) * w).sum().backward()
    wn = w.cpu().double().numpy()
    mg_want = mg64 * wn[:, None, None]
    lg_want = lg64 * wn[:, None, None, None]
    mg_got, lg_got = md.grad.cpu().double().numpy(), ld.grad.cpu().double().numpy()
    assert np.isfinite(mg_got).all() and np.isfinite(lg_got).all()
    worst = np.zeros((2, len(gradcheck.BANDS)))
    for bi in range(len(wn)):
        scale = max(np.abs(mg_want[bi]).max(), 1e-30)
        assert np.abs(mg_got[bi] - mg_want[bi]).max() <= 1e-4 * scale, (case, bi)
        scale = max(np.abs(lg_want[bi]).max(), 1e-30)
        assert np.abs(lg_got[bi] - lg_want[bi]).max() <= 1e-4 * scale, (case, bi)
        if not fin[bi]:
            assert not mg_got[bi].any() and not lg_got[bi].any()
        # every entry, relative to its own size
        worst[0] = np.maximum(worst[0], gradcheck.assert_elementwise(mg_got[bi], mg_want[bi], "%s: match_all_grad of sentence %d" % (case, bi)))
        worst[1] = np.maximum(worst[1], gradcheck.assert_elementwise(lg_got[bi], lg_want[bi], "%s: links_grad of sentence %d" % (case, bi)))
    print("%s: worst relative error of an entry, by its share of the sentence maximum (%s): match_all_grad %s, links_grad %s"
          % (case, ", ".join(">= %.0e" % f for f, _ in gradcheck.BANDS), " ".join("%.1e" % e for e in worst[0]),
             " ".join("%.1e" % e for e in worst[1])))


def _inside_all(batch, match):
    md = match.to(DEV).requires_grad_(True)
    ld = batch["links"].to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, batch["output_length"].to(DEV), batch["target_length"].to(DEV))
    w = torch.linspace(0.5, 1.5, ll.numel(), device=DEV)
    (ll.masked_fill(~torch.isfinite(ll), 0) * w).sum().backward()
    return ll.detach().cpu(), md.grad.cpu(), ld.grad.cpu()


def test_sentence_given_up_is_counted_and_invalid():
    """Where both pipelined sweeps of a sentence give up (spin limit 0) and the second chance of the outside sweep also
    runs out of its bound for the forward's (forced: a bound of zero polls, so the wait expires without waiting), the
    sentence is given up: NaN log-likelihood, zero gradients, and the third diagnostic counter says how many - a valid
    sentence never turns invalid unnoticed.  The default path leaves that counter at zero (test_long_graph_sweeps_agree)."""
    L, T, ms, ns = 320, 40, [320, 262, 200], [40, 31, 25]
    batch = synth.training_batch(len(ms), L, T, 60, ms, ns, seed=L + T)
    match = _match_for(batch)
    ll0, mg0, lg0 = _inside_all(batch, match)
    assert torch.isfinite(ll0).all()
    ops.pipeline_redo_counts(reset=True)
    try:
        ops.pipeline_config(spin_limit=0)
        ops.pipeline_redo_wait_limit(0)
        ll1, mg1, lg1 = _inside_all(batch, match)
    finally:
        ops.pipeline_config(max_workgroups=1 << 20, spin_limit=ops.DEFAULT_SPIN_LIMIT, outside_spin_limit=-1)
        ops.pipeline_redo_wait_limit()
    redone, _, given_up = ops.pipeline_redo_counts(reset=True)
    bad = torch.isnan(ll1)
    assert given_up == int(bad.sum()), (given_up, ll1)
    assert given_up >= 1, "no sentence had both of its sweeps give up: the case was not exercised"
    for b in range(len(ms)):
        if bad[b]:
            assert not mg1[b].any() and not lg1[b].any()
        else:
            assert torch.allclose(ll1[b], ll0[b], rtol=1e-5)
            assert (mg1[b] - mg0[b]).abs().max() <= 2e-5 * mg0[b].abs().max()


@pytest.mark.parametrize("mode", ["one_workgroup", "blocks_give_up", "pipelines_in_turn", "forward_gives_up", "outside_gives_up"])
@pytest.mark.parametrize("L,T,ms,ns", [(200, 50, [200, 132, 164], [50, 30, 44]), (320, 40, [320, 262, 4], [40, 31, 2]),
                                       (512, 140, [512, 444], [140, 120]),
                                       (600, 24, [600, 520], [24, 24]), (1024, 30, [1024, 770, 900], [30, 22, 30]),
                                       (130, 30, [130, 128, 66], [30, 30, 17]),
                                       # more blocks than compute units: the blocks share them (one collector wave each)
                                       (200, 20, [200, 132, 164, 96] * 10, [20, 13, 17, 9] * 10),
                                       # a large batch: 4096 blocks per pipeline, sixteen times the compute units
                                       (512, 24, [512, 444, 386, 512] * 64, [24, 21, 24, 18] * 64)])
def test_long_graph_sweeps_agree(mode, L, T, ms, ns):
    """Graphs of 130..1026 nodes: the two pipelined sweeps side by side (default), one after the other (a workgroup budget
    that holds one pipeline but not two), the one-workgroup streaming sweeps (pipeline switched off) and the redo path
    (blocks that give up at once: spin limit 0; both sweeps, or only one of the two that run side by side) compute the
    same tables; the default path is compared with the oracle in test_inside_forward_backward_vs_oracle."""
    batch = synth.training_batch(len(ms), L, T, 60, ms, ns, seed=L + T)
    match = _match_for(batch)
    ops.pipeline_redo_counts(reset=True)
    ll0, mg0, lg0 = _inside_all(batch, match)
    counts = ops.pipeline_redo_counts()
    assert counts[0] == 0 and counts[2] == 0, "the pipelined sweeps of the default path gave up: %s" % (counts,)
    try:
        if mode == "one_workgroup":
            ops.pipeline_config(max_workgroups=0)
        elif mode == "pipelines_in_turn":
            ops.pipeline_config(max_workgroups=len(ms) * 4 * ((L // 2 + 63) // 64))
        elif mode == "forward_gives_up":  # ... and is redone, while the outside pipeline beside it completes
            ops.pipeline_config(spin_limit=0, outside_spin_limit=ops.DEFAULT_SPIN_LIMIT)
        elif mode == "outside_gives_up":
            ops.pipeline_config(outside_spin_limit=0)
        else:
            ops.pipeline_config(spin_limit=0)
        ll1, mg1, lg1 = _inside_all(batch, match)
    finally:
        ops.pipeline_config(max_workgroups=1 << 20, spin_limit=ops.DEFAULT_SPIN_LIMIT, outside_spin_limit=-1)
    # the fallback is visible in the diagnostic counter: every sweep of every sentence that ran as a pipeline and gave up
    # (a block gives up only if it has to wait at all, so how many sentences are redone varies from run to run)
    redone, _, given_up = ops.pipeline_redo_counts(reset=True)
    assert given_up == 0, "a second chance ran out of its bound"
    if mode in ("one_workgroup", "pipelines_in_turn"):
        assert redone == 0, (mode, redone)
    else:
        most = len(ms) * (2 if mode == "blocks_give_up" else 1)
        assert 0 < redone <= most, (mode, redone, most)
    fin = torch.isfinite(ll0)
    assert fin.any() and torch.equal(fin, torch.isfinite(ll1))
    assert torch.allclose(ll0[fin], ll1[fin], rtol=1e-5)
    for b in range(len(ms)):
        for g0, g1 in ((mg0[b], mg1[b]), (lg0[b], lg1[b])):
            assert (g0 - g1).abs().max() <= 1e-4 * max(g0.abs().max().item(), 1e-30)


@pytest.mark.parametrize("case", ["L130", "L256", "L320_mixed", "L512_long", "L1028"])
def test_rule_posteriors_term_by_term_path(case):
    """The rule posteriors of long graphs with every tile sent down the path without a range limit (one exponential per
    term instead of the factored sum on the matrix cores): same gradients, against the float64 oracle."""
    try:
        ops.links_grad_range_limit(float("-inf"))
        test_inside_forward_backward_vs_oracle(case)
    finally:
        ops.links_grad_range_limit()


def test_inside_extreme_inputs_vs_oracle():
    """Of four sentences one has an emission 400 nats down, one a link 300 nats down, one a node whose inside value falls
    2^-600 below its column's largest, one nothing special: every sentence comes out right against the float64 oracle (the
    sweeps work in the log domain relative to per-column offsets, so none of this leaves their range)."""
    L, T, ms, ns = 64, 20, [64, 64, 64, 64], [20, 20, 20, 20]
    batch = synth.training_batch(4, L, T, 80, ms, ns, seed=77)
    match = _match_for(batch).clone()
    links = batch["links"].clone()
    match[0, 9, 5] = -400.0
    fin = torch.isfinite(links[1, 5, 0])
    links[1, 5, 0, int(fin.nonzero()[0])] = -300.0
    match[2, 41:, :] = match[2, 41:, :] - 90.0  # every emission of the right part of the graph: 5 tokens are 2^-650
    batch = dict(batch, links=links)
    S64, C64, mg64, lg64 = _oracle_inside(batch, match.numpy())
    ll, mg, lg = _inside_all(batch, match)
    w = torch.linspace(0.5, 1.5, 4).double().numpy()
    assert np.allclose(ll.double().numpy(), S64[:, 0, 0], rtol=1e-5)
    for bi in range(4):
        for got, want in ((mg[bi].double().numpy(), mg64[bi] * w[bi]), (lg[bi].double().numpy(), lg64[bi] * w[bi])):
            assert np.abs(got - want).max() <= 1e-4 * max(np.abs(want).max(), 1e-30), bi


@pytest.mark.parametrize("wrong", [-16.0, -24.0, -32.0])
def test_inside_peaked_emissions_vs_oracle(wrong):
    """Peaked emissions, as a trained model gives them: every token has one node that emits it with probability 0.8, all
    other nodes are `wrong` nats down.  A node far from the alignment then falls more than 2^-500 below its column's
    largest after some tokens.  Loss, table and gradients against the float64 oracle."""
    L, T = 128, 32
    ms, ns = [128, 128, 96, 64, 40, 128], [32, 30, 25, 17, 11, 9]
    batch = synth.training_batch(len(ms), L, T, 80, ms, ns, seed=41)
    g = torch.Generator().manual_seed(int(-wrong))
    match = wrong + 2.0 * torch.randn(len(ms), L, T, generator=g)
    for b, (m, n) in enumerate(zip(ms, ns)):
        for t in range(n):
            a = 2 * int(round(t * (m // 2 - 1) / max(n - 1, 1))) + 1
            match[b, min(a, m - 1), t] = -0.2
    match = harness.eos_masked(match, batch["output_length"], batch["target_length"])
    assert float(match[torch.isfinite(match)].min()) > -100.0
    S64, C64, mg64, lg64 = _oracle_inside(batch, match.numpy())
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    ll, mg, lg = _inside_all(batch, match)
    S = ops._pcfg_loss_tables(match.to(DEV), batch["links"].to(DEV), ol, tl, 1, "test")[0].cpu().double().numpy()
    assert np.array_equal(np.isneginf(S), np.isneginf(S64))
    fin = np.isfinite(S64)
    assert np.allclose(S[fin], S64[fin], rtol=2e-6, atol=1e-4)
    assert np.allclose(ll.double().numpy(), S64[:, 0, 0], rtol=1e-5)
    w = torch.linspace(0.5, 1.5, len(ms)).double().numpy()
    for bi in range(len(ms)):
        for got, want in ((mg[bi].double().numpy(), mg64[bi] * w[bi]), (lg[bi].double().numpy(), lg64[bi] * w[bi])):
            assert np.abs(got - want).max() <= 1e-4 * max(np.abs(want).max(), 1e-30), bi


@pytest.mark.parametrize("n,width", [(16, 4), (16, 6), (16, 1), (5, 1), (4, 1), (3, 1), (2, 1)])
def test_inside_emissions_that_collapse_at_every_column_vs_oracle(n, width):
    """One sentence per column p: `width` consecutive tokens from p on are emitted with probability e^-95 by every node but
    one, so the spread of the columns grows by 137 bits a token there - at a column that moves with p from the first step
    of either sweep to its last; sentences of two to five tokens put every such case next to the ends of the sweeps.
    Everything against the float64 oracle."""
    L, T = 64, 16
    cases = list(range(0, max(n - width, 0) + 1))
    ms, ns = [64 - 2 * (p % 3) for p in cases], [n] * len(cases)
    batch = synth.training_batch(len(cases), L, T, 80, ms, ns, seed=5 * n + width)
    g = torch.Generator().manual_seed(n + width)
    match = -3.0 + torch.randn(len(cases), L, T, generator=g)
    for b, (p0, m) in enumerate(zip(cases, ms)):
        for t in range(p0, min(p0 + width, n)):
            a = 2 * int(round(t * (m // 2 - 1) / max(n - 1, 1))) + 1
            keep = match[b, min(a, m - 1), t].clone()
            match[b, :, t] -= 95.0
            match[b, min(a, m - 1), t] = keep
    match = harness.eos_masked(match, batch["output_length"], batch["target_length"])
    assert float(match[torch.isfinite(match)].min()) > -103.0
    S64, C64, mg64, lg64 = _oracle_inside(batch, match.numpy())
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    ll, mg, lg = _inside_all(batch, match)
    S = ops._pcfg_loss_tables(match.to(DEV), batch["links"].to(DEV), ol, tl, 1, "test")[0].cpu().double().numpy()
    assert np.array_equal(np.isneginf(S), np.isneginf(S64))
    fin = np.isfinite(S64)
    assert np.allclose(S[fin], S64[fin], rtol=2e-6, atol=1e-4)
    assert np.allclose(ll.double().numpy(), S64[:, 0, 0], rtol=1e-5)
    w = torch.linspace(0.5, 1.5, len(cases)).double().numpy() if len(cases) > 1 else np.array([0.5])
    for bi in range(len(cases)):
        for got, want in ((mg[bi].double().numpy(), mg64[bi] * w[bi]), (lg[bi].double().numpy(), lg64[bi] * w[bi])):
            assert np.abs(got - want).max() <= 1e-4 * max(np.abs(want).max(), 1e-30), bi


@pytest.mark.parametrize("L,T,ms,ns", [(128, 30, [128, 90], [30, 22]), (320, 40, [320, 262], [40, 31]), (600, 24, [600, 520], [24, 24])])
def test_inside_spiky_inputs_vs_oracle(L, T, ms, ns):
    """Emissions and links with jumps of hundreds of units and scattered -inf entries: neighbouring columns of the tables
    then differ by far more than one token's log-probability, which is what the streaming sweeps' guessed shifts (and
    the column offsets of all sweeps) must survive.  Whole S table (including its -inf pattern) and both gradients
    against the float64 oracle."""
    batch = synth.training_batch(len(ms), L, T, 60, ms, ns, seed=L + T)
    g = torch.Generator().manual_seed(5 * L + 1)
    match = _match_for(batch)
    u = torch.rand(match.shape, generator=g)
    match = match - 300.0 * (u < 0.3) - 700.0 * (u > 0.93)
    match = match.masked_fill(torch.rand(match.shape, generator=g) < 0.03, float("-inf"))
    links = batch["links"].clone()
    v = torch.rand(links.shape, generator=g)
    links = links - 250.0 * (v < 0.2)
    links = links.masked_fill(torch.rand(links.shape, generator=g) < 0.05, float("-inf"))
    batch = dict(batch, links=links)
    S64, C64, mg64, lg64 = _oracle_inside(batch, match.numpy())
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    S, _, _, _ = ops._pcfg_loss_tables(match.to(DEV), links.to(DEV), ol, tl, 1, "test")
    S = S.cpu().double().numpy()
    assert np.array_equal(np.isneginf(S), np.isneginf(S64))
    fin = np.isfinite(S64)
    assert np.isfinite(S64[:, 0, 0]).any()
    assert np.allclose(S[fin], S64[fin], rtol=2e-6, atol=1e-4)
    md, ld = match.to(DEV).requires_grad_(True), links.to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, ol, tl)
    ll.masked_fill(~torch.isfinite(ll), 0).sum().backward()
    mg_got, lg_got = md.grad.cpu().double().numpy(), ld.grad.cpu().double().numpy()
    assert np.isfinite(mg_got).all() and np.isfinite(lg_got).all()
    for bi in range(len(ms)):
        if not np.isfinite(S64[bi, 0, 0]):
            assert not mg_got[bi].any() and not lg_got[bi].any()
            continue
        assert np.abs(mg_got[bi] - mg64[bi]).max() <= 1e-4 * np.abs(mg64[bi]).max(), bi
        assert np.abs(lg_got[bi] - lg64[bi]).max() <= 1e-4 * np.abs(lg64[bi]).max(), bi


def test_inside_tables_match_oracle_layout():
    batch = _train_case("ragged_short")
    match = _match_for(batch)
    S64, _, _, _ = _oracle_inside(batch, match.numpy())
    S, aux, _, _ = ops._pcfg_loss_tables(match.to(DEV), batch["links"].to(DEV), batch["output_length"].to(DEV),
                                         batch["target_length"].to(DEV), 1, "test")
    S = S.cpu().double().numpy()
    assert S.shape == S64.shape
    assert np.array_equal(np.isneginf(S), np.isneginf(S64))
    fin = np.isfinite(S64)
    assert np.allclose(S[fin], S64[fin], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("case", ["cfg1", "wmt_small", "ragged_short", "L256", "L512", "L512_long"])
def test_best_tree_bit_exact(case):
    batch = _train_case(case)
    match = _match_for(batch)
    links = batch["links"]
    ol, tl = batch["output_length"], batch["target_length"]
    tree, ll = ops.cuda_pcfg_best_tree(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV))
    assert tree.dtype == torch.int64 and not tree.requires_grad
    S_gpu, _, _, _ = ops._pcfg_loss_tables(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV), 1, "test")
    S64, C64 = oracle.inside_fwd(match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float32)
    # the trace of the oracle fed with the very tables the GPU trace saw: must agree bit for bit
    want = oracle.best_tree(S_gpu.cpu().numpy(), C64, match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float32)
    assert np.array_equal(tree.cpu().numpy(), want)
    # and the trace over the oracle's own float64 tables is the same alignment on these inputs
    S64d, C64d = oracle.inside_fwd(match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float64)
    want64 = oracle.best_tree(S64d, C64d, match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float64)
    assert np.array_equal(tree.cpu().numpy(), want64)
    for bi in range(tree.shape[0]):
        if math.isfinite(float(ll[bi])):
            used = tree[bi][tree[bi] >= 0].cpu().tolist()
            assert used == list(range(int(tl[bi])))


def test_best_tree_exact_ties_follow_reference_order():
    L = m = 14
    n = 3
    links = torch.full((1, L, 2, L), -math.inf)
    for a in range(1, m - 1, 2):
        links[0, a, 0, a + 2:m:2] = -1.0
    match = torch.full((1, L, n), -1.0)
    ol, tl = torch.tensor([m]), torch.tensor([n])

    def second(dead):
        lk = links.clone()
        for cid in dead:
            lk[0, 1, 0, 2 * cid + 1] = -math.inf
        tree, _ = ops.cuda_pcfg_best_tree(match.to(DEV), lk.to(DEV), ol.to(DEV), tl.to(DEV))
        pos = (tree[0] == 1).nonzero().item()
        return (pos - 1) // 2

    assert second(()) == 1
    assert second((1,)) == 5
    assert second((1, 5)) == 3
    assert second((1, 5, 3)) == 2
    assert second((1, 5, 3, 2)) == 4


@pytest.mark.parametrize("ml", [1, 3])
def test_glat_single_call_small_ragged(ml):
    """Ragged small batch (one sentence whose target cannot be derived) through the one-call GLAT pass against the torch
    glue over the oracle ops, for the tuned (max_left 1) and the general kernels."""
    import oracle_ops
    g = torch.Generator().manual_seed(40 + ml)
    L, T, V = 8 * (ml + 1) + 2, 9, 97
    ms = [L, L - 2 * (ml + 1), (ml + 1) * 2 + 2, L]
    ns = [9, 6, 9, 7]  # sentence 2: nine tokens from three main-chain nodes, impossible
    B = len(ms)
    m = torch.tensor(ms)
    links = synth.make_links(B, L, m, ml, g)
    tgt = torch.full((B, T), synth.PAD, dtype=torch.int64)
    for b, n in enumerate(ns):
        tgt[b, :n] = torch.randint(4, V, (n,), generator=g)
    prev = torch.full((B, L), 3, dtype=torch.int64).masked_fill(torch.arange(L).view(1, L) >= m.view(B, 1), synth.PAD)
    logits = torch.randn(B, L, V, generator=g)
    for b in range(B):  # let some predictions agree with the targets
        logits[b, 1, tgt[b, 0]] += 20.0
    g1, g2 = torch.Generator().manual_seed(5), torch.Generator().manual_seed(5)
    want = harness.glat_alignment(logits.clone(), tgt, prev, links, 0.5, ops=oracle_ops, generator=g1)
    got = harness.glat_alignment(logits.to(DEV), tgt.to(DEV), prev.to(DEV), links.to(DEV), 0.5, generator=g2, noise_device="cpu",
                                 single_call=True)
    for key in ("path", "keep_word_mask", "glat_prev_output_tokens", "matchmask", "same_num", "glance_nums"):
        assert got[key].dtype == want[key].dtype and torch.equal(got[key].cpu(), want[key]), key
    assert int(want["same_num"].sum()) >= 1
    assert torch.allclose(got["max_tree_lprob"].cpu(), want["max_tree_lprob"], rtol=2e-5)


@pytest.mark.parametrize("case", ["wmt_small", "L130", "L256", "L512_long"])
@pytest.mark.parametrize("strategy", ["number-random", None])
def test_glat_single_call_on_longer_graphs(case, strategy):
    """The one-call GLAT pass (best tree and glue by one workgroup per sentence) against the torch glue over the separate
    device operators with the same random numbers, on graphs whose link matrices or whose tables no longer fit the
    workgroup's LDS beside each other (the walk then reads them from memory); the separate operators are held against the
    oracle by the tests above."""
    batch = _train_case(case)
    logits, tgt, links = batch["logits"].to(DEV), batch["targets"].to(DEV), batch["links"].to(DEV)
    B, L, _ = logits.shape
    prev = torch.full((B, L), 3, dtype=torch.int64)
    prev = prev.masked_fill(torch.arange(L).view(1, L) >= batch["output_length"].view(B, 1), synth.PAD).to(DEV)
    g1, g2 = torch.Generator().manual_seed(11), torch.Generator().manual_seed(11)
    want = harness.glat_alignment(logits, tgt, prev, links, 0.5, generator=g1, noise_device="cpu", glance_strategy=strategy)
    got = harness.glat_alignment(logits, tgt, prev, links, 0.5, generator=g2, noise_device="cpu", glance_strategy=strategy,
                                 single_call=True)
    for key in ("path", "keep_word_mask", "glat_prev_output_tokens", "matchmask", "same_num", "glance_nums"):
        assert got[key].dtype == want[key].dtype and torch.equal(got[key], want[key]), key
    assert torch.allclose(got["max_tree_lprob"], want["max_tree_lprob"], rtol=2e-5)
    assert int((got["path"] >= 0).sum()) > 0


@pytest.mark.parametrize("B,L,H,F,dtype", [(3, 18, 2, 4, torch.float32), (2, 34, 8, 16, torch.float32), (4, 128, 8, 64, torch.float16),
                                            (2, 514, 4, 8, torch.float32), (2, 22, 16, 8, torch.float32), (2, 12, 1, 8, torch.float32),
                                            (2, 200, 4, 16, torch.float16), (2, 256, 2, 24, torch.float32), (3, 130, 8, 64, torch.float32),
                                            (2, 66, 16, 32, torch.float16), (2, 96, 2, 64, torch.float16)])
@pytest.mark.parametrize("products_inside", [True, False])
def test_extract_links_forward_backward_vs_torch_restatement(B, L, H, F, dtype, products_inside):
    """Both forms of the scorer (products on the matrix cores inside the kernels where the shape is covered; products
    through torch's GEMM library) against the float64 restatement: links and all four gradients."""
    from oracle import extract_links_ref as ref
    g = torch.Generator().manual_seed(L + H)
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 0.7).to(dtype) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).to(dtype)
    ms = [L, max(4, (L // 2) // 2 * 2), 4, L][:B]
    m = torch.tensor(ms)
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= m.view(B, 1), synth.PAD)
    lm, rm, mc = synth.support_masks(L, 1)
    leaves = [t.double().requires_grad_(True) for t in (q, kl, kr, gate)]
    want = ref.extract_links(*leaves, prev, synth.PAD, lm, rm, mc).double()
    fin = torch.isfinite(want)
    G = torch.randn(want.shape, generator=g, dtype=torch.float64).masked_fill(~fin, 0)
    want.masked_fill(~fin, 0).mul(G).sum().backward()
    dleaves = [t.to(DEV).requires_grad_(True) for t in (q, kl, kr, gate)]
    got = ops.pcfg_extract_links(*dleaves, prev.to(DEV), synth.PAD, lm.to(DEV), rm.to(DEV), mc.to(DEV), products_inside)
    assert got.dtype == torch.float32 and torch.equal(torch.isfinite(got).cpu(), fin)
    assert torch.allclose(got.cpu().double()[fin], want.detach()[fin], rtol=2e-5, atol=2e-5)
    got.masked_fill(~fin.to(DEV), 0).mul(G.float().to(DEV)).sum().backward()
    for name, mine, theirs in zip(("q", "kl", "kr", "gate"), dleaves, leaves):
        assert mine.grad.dtype == dtype
        scale = theirs.grad.abs().max().item()
        err = (mine.grad.cpu().double() - theirs.grad).abs().max().item()
        tol = 2e-3 if dtype == torch.float16 else 1e-4
        assert err <= tol * scale, (name, err, scale)


@pytest.mark.parametrize("B,L,H,F,dtype", [(2, 34, 8, 16, torch.float32), (4, 128, 8, 64, torch.float16), (2, 514, 4, 8, torch.float32),
                                            (2, 22, 16, 8, torch.float32), (2, 12, 1, 8, torch.float32), (2, 200, 4, 16, torch.float16),
                                            (3, 130, 8, 64, torch.float32), (2, 66, 16, 32, torch.float16), (2, 40, 2, 128, torch.float16)])
def test_extract_links_products_inside_the_kernel(B, L, H, F, dtype):
    """The scorer's forward with its three products on the matrix cores inside the kernel, also at head dimension 128
    (where only the forward is built): links against the float64 restatement and against the five-call form, graphs that
    are no multiple of the 32-wide tiles, padded sentences, 1 to 16 heads."""
    from oracle import extract_links_ref as ref
    lib = ops.get_pcfg_kernel()
    assert lib.pcfgnat_extract_links_fused_supported(ops._DTYPE_CODE[dtype], L, H, F) == 1
    g = torch.Generator().manual_seed(L + H)
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 0.7).to(dtype) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).to(dtype)
    ms = [L, max(4, (L // 2) // 2 * 2), 4, L][:B]
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= torch.tensor(ms).view(B, 1), synth.PAD)
    lm, rm, mc = synth.support_masks(L, 1)
    want = ref.extract_links(*(t.double() for t in (q, kl, kr, gate)), prev, synth.PAD, lm, rm, mc).double()
    fin = torch.isfinite(want)
    dev = [t.to(DEV) for t in (q, kl, kr, gate)]
    with torch.no_grad():
        got = ops.pcfg_extract_links(*dev, prev.to(DEV), synth.PAD, lm.to(DEV), rm.to(DEV), mc.to(DEV))
    assert got.dtype == torch.float32 and torch.equal(torch.isfinite(got).cpu(), fin)
    assert torch.allclose(got.cpu().double()[fin], want[fin], rtol=2e-5, atol=2e-5)
    # the five-call form gives the same links
    with torch.no_grad():
        other = ops.pcfg_extract_links(*dev, prev.to(DEV), synth.PAD, lm.to(DEV), rm.to(DEV), mc.to(DEV), False)
    assert torch.equal(torch.isfinite(other), torch.isfinite(got))
    assert torch.allclose(got[fin.to(DEV)], other[fin.to(DEV)], rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("B,L,H,F,dtype,ms", [(1, 2, 2, 16, torch.float16, [2]), (2, 3, 4, 8, torch.float32, [3, 2]),
                                               (3, 6, 8, 16, torch.float16, [6, 0, 4]), (1, 70, 16, 64, torch.float16, [66]),
                                               (2, 33, 1, 64, torch.float32, [33, 32])])
def test_extract_links_products_inside_edge_shapes(B, L, H, F, dtype, ms):
    """The smallest graphs, a single sentence, a sentence that is all pad, sixteen heads of 64, a tile boundary at 32 + 1
    nodes: links and gradients of the form with the products inside against the form with the products through torch."""
    g = torch.Generator().manual_seed(7 * L + H)
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 0.7).to(dtype).to(DEV) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).to(dtype).to(DEV)
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= torch.tensor(ms).view(B, 1), synth.PAD).to(DEV)
    lm, rm, mc = (t.to(DEV) for t in synth.support_masks(L, 1))
    G = torch.randn(B, L, 2, L, generator=g).to(DEV)
    res = []
    for inside in (True, False):
        leaves = [t.clone().requires_grad_(True) for t in (q, kl, kr, gate)]
        out = ops.pcfg_extract_links(*leaves, prev, synth.PAD, lm, rm, mc, inside)
        fin = torch.isfinite(out)
        out.masked_fill(~fin, 0).mul(G).sum().backward()
        res.append((out.detach(), [t.grad for t in leaves]))
    (a, ga), (b, gb) = res
    assert torch.equal(torch.isfinite(a), torch.isfinite(b))
    fin = torch.isfinite(a)
    assert torch.allclose(a[fin], b[fin], rtol=2e-5, atol=2e-5)
    for name, x, y in zip(("q", "kl", "kr", "gate"), ga, gb):
        assert torch.isfinite(x).all(), name
        scale = max(y.float().abs().max().item(), 1e-6)
        tol = 4e-3 if dtype == torch.float16 else 1e-4  # fp16: both results are rounded to the chunks' dtype
        assert (x.float() - y.float()).abs().max().item() <= tol * scale, name


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_extract_links_products_inside_keeps_links_far_below_float_range(dtype):
    """Sharp heads: many links come out hundreds of nats below zero, where every head's share of the entry is below the
    smallest float.  The mixture over the heads, formed as a plain sum of probabilities where that is safe, must take such
    entries through the shifted form and return the logarithm the float64 restatement has - finite, not -inf."""
    from oracle import extract_links_ref as ref
    g = torch.Generator().manual_seed(123)
    B, L, H, F = 2, 96, 2, 64
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 8).to(dtype) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).to(dtype)
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= torch.tensor([L, 70]).view(B, 1), synth.PAD)
    lm, rm, mc = synth.support_masks(L, 1)
    want = ref.extract_links(q.double(), kl.double(), kr.double(), gate.double(), prev, synth.PAD, lm, rm, mc).double()
    fin = torch.isfinite(want)
    assert (want[fin] < -100).sum() > 100 and (want[fin] < -200).any()   # far below log(2^-126) = -87.3
    got = ops.pcfg_extract_links(q.to(DEV), kl.to(DEV), kr.to(DEV), gate.to(DEV), prev.to(DEV), synth.PAD, lm.to(DEV), rm.to(DEV),
                                 mc.to(DEV))
    assert torch.equal(torch.isfinite(got).cpu(), fin)
    assert torch.allclose(got.cpu().double()[fin], want[fin], rtol=2e-5, atol=2e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_extract_links_products_inside_arbitrary_masks(dtype):
    """The backward leaves out the tiles of 32 x 32 (parent, right child) pairs in which the masks allow nothing and runs
    over the range of tiles that hold pairs, which it finds from the masks alone: tree masks that are no triangle (allowed
    right children in front of their parents), a band of right children that no parent may take (a hole in the middle of
    the range), parents without any allowed right child, pad nodes behind the sentences - against the form with the
    products through torch, which knows no tiles."""
    g = torch.Generator().manual_seed(99)
    B, L, H, F = 3, 162, 4, 16  # six tiles, the last one partial
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 0.7).to(dtype).to(DEV) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).to(dtype).to(DEV)
    ms = [L, 100, 40]
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= torch.tensor(ms).view(B, 1), synth.PAD).to(DEV)
    rm = (torch.rand(L, L, generator=g) > 0.15).long()   # 1 = forbidden: about 15 % of the pairs allowed, anywhere
    rm[:, 64:96] = 1                                     # no parent may take a right child of the third tile
    rm[32:64, :32] = 0                                   # the second tile of parents: every child of the first tile
    rm[96:100, :] = 1                                    # a few parents without a right child
    lm = (torch.rand(L, L, generator=g) > 0.5).long()
    lm[:, 0] = 0                                         # node 0 may be everybody's left child
    mc = torch.ones(L, dtype=torch.bool)
    lm, rm, mc = lm.to(DEV), rm.to(DEV), mc.to(DEV)
    G = torch.randn(B, L, 2, L, generator=g).to(DEV)
    res = []
    for inside in (True, False):
        leaves = [t.clone().requires_grad_(True) for t in (q, kl, kr, gate)]
        out = ops.pcfg_extract_links(*leaves, prev, synth.PAD, lm, rm, mc, inside)
        fin = torch.isfinite(out)
        out.masked_fill(~fin, 0).mul(G).sum().backward()
        res.append((out.detach(), [t.grad for t in leaves]))
    (a, ga), (b, gb) = res
    fin = torch.isfinite(a)
    assert torch.equal(fin, torch.isfinite(b)) and fin.any() and not fin[:, :, :, 64:96].any()
    assert fin[0, 32:64, :, :32].any()                   # links to right children in front of the parents
    assert torch.allclose(a[fin], b[fin], rtol=2e-5, atol=2e-5)
    for name, x, y in zip(("q", "kl", "kr", "gate"), ga, gb):
        assert torch.isfinite(x).all(), name
        scale = max(y.float().abs().max().item(), 1e-6)
        tol = 4e-3 if dtype == torch.float16 else 1e-4
        assert (x.float() - y.float()).abs().max().item() <= tol * scale, name


def test_extract_links_fused_form_rejects_what_it_does_not_cover():
    lib = ops.get_pcfg_kernel()
    assert lib.pcfgnat_extract_links_fused_supported(ops._DTYPE_CODE[torch.float32], 256, 2, 24) == 0   # head dimension
    assert lib.pcfgnat_extract_links_fused_supported(ops._DTYPE_CODE[torch.float64], 64, 2, 16) == 0    # dtype
    assert lib.pcfgnat_extract_links_fused_supported(ops._DTYPE_CODE[torch.float16], 64, 3, 16) == 0    # heads
    assert lib.pcfgnat_extract_links_fused_supported(ops._DTYPE_CODE[torch.float32], 64, 16, 64) == 0   # tile rows beyond the LDS
    assert lib.pcfgnat_extract_links_fused_backward_supported(ops._DTYPE_CODE[torch.float16], 64, 2, 128) == 0  # backward: up to 64
    assert lib.pcfgnat_extract_links_fused_backward_supported(ops._DTYPE_CODE[torch.float16], 64, 2, 64) == 1
    x = torch.zeros(1, 64, 3, 16, device=DEV, dtype=torch.float16)
    rc = lib.pcfgnat_extract_links_fused_forward(x.data_ptr(), x.data_ptr(), x.data_ptr(), ops._DTYPE_CODE[torch.float16], x.data_ptr(),
                                                 x.data_ptr(), 1, x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(),
                                                 None, 1, 64, 3, 16, None)
    assert rc != 0 and b"heads" in lib.pcfgnat_last_error()


def _decode_case(name):
    if name == "short":
        return synth.decode_batch([5, 9, 16, 3, 12], seed=3, V=500)
    if name == "L256":
        return synth.decode_batch([64, 40, 33], seed=4, V=300)
    if name == "L400":  # longest graph of the inference configuration: widest register-resident slabs but one
        return synth.decode_batch([100, 71, 5], seed=6, V=100)
    if name == "L512":  # widest register-resident slabs
        return synth.decode_batch([128, 117, 20], seed=7, V=64)
    if name == "L600":  # beyond the register-resident kernels: streaming kernel
        return synth.decode_batch([150, 90], seed=8, V=64)
    if name in ("L96", "L160", "L224", "L288", "L352"):  # one case per slab width in between
        n = int(name[1:]) // 4
        return synth.decode_batch([n, n - 3, 7], seed=n, V=64)
    raise KeyError(name)


@pytest.mark.parametrize("case", ["short", "L96", "L160", "L224", "L256", "L288", "L352", "L400", "L512", "L600"])
def test_viterbi_tables_bit_exact_and_decode(case):
    batch = _decode_case(case)
    ob, tok = synth.ob_and_tokens(batch["logits"])
    links, ol = batch["links"], batch["output_length"]
    L = links.shape[1]
    scores, R, Lt, M = ops.cuda_pcfg_viterbi(ob.to(DEV), links.to(DEV), ol.to(DEV))
    S_o, R_o, L_o, M_o = oracle.viterbi(ob.numpy(), links.numpy(), ol.numpy(), dtype=np.float32)
    assert scores.shape == (links.shape[0], L // 4)
    assert np.array_equal(scores.cpu().numpy(), S_o[:, 1, :])  # bit-exact, -inf included
    assert np.array_equal(R.cpu().numpy(), R_o)
    assert np.array_equal(Lt.cpu().numpy(), L_o)
    assert np.array_equal(M.cpu().numpy(), M_o)
    left_mask, _, _ = synth.support_masks(L, 1)
    # glue + readout, traces on the device and on the host, against the same glue over the oracle
    import oracle_ops
    want_tok, want_len = harness.viterbi_decode(ob, tok, links, ol, left_mask, ops=oracle_ops)
    for on_host in (False, True):
        got_tok, got_len = harness.viterbi_decode(ob.to(DEV), tok.to(DEV), links.to(DEV), ol.to(DEV), left_mask.to(DEV),
                                                  traces_on_host=on_host)
        assert torch.equal(got_len.cpu(), want_len)
        assert got_tok.dtype == torch.float32 and torch.equal(got_tok.cpu(), want_tok)
    # the whole decode as one native call, with and without a length penalty exponent
    for beta in (1.0, 0.7):
        want_tok, want_len = harness.viterbi_decode(ob, tok, links, ol, left_mask, ops=oracle_ops, beta=beta)
        got_tok, got_len = harness.viterbi_decode(ob.to(DEV), tok.to(DEV), links.to(DEV), ol.to(DEV), left_mask.to(DEV),
                                                  beta=beta, single_call=True)
        assert got_len.dtype == torch.int64 and torch.equal(got_len.cpu(), want_len)
        assert got_tok.dtype == torch.float32 and torch.equal(got_tok.cpu(), want_tok)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("case", ["short", "L96", "L224", "L400", "L600"])
def test_decode_from_logits_is_front_end_plus_decode(case, dtype):
    """The call that takes the vocabulary logits returns, bit for bit, what the front-end followed by the decode returns
    (the same kernels enqueued by one call), node scores and node tokens included; the decode itself is held against the
    oracle by the tests above."""
    batch = _decode_case(case)
    logits = batch["logits"].to(dtype).to(DEV).contiguous()
    links, ol = batch["links"].to(DEV), batch["output_length"].to(DEV)
    left_mask = synth.support_masks(links.shape[1], 1)[0].to(DEV)
    for beta in (1.0, 0.7):
        ob, tok = ops.logsoftmax_max(logits)
        want_tok, want_len = ops.pcfg_viterbi_decode(ob, links, ol, tok, left_mask, synth.PAD, beta)
        got_tok, got_len, got_ob, got_nodes = ops.pcfg_viterbi_decode_logits(logits, links, ol, left_mask, synth.PAD, beta,
                                                                             return_nodes=True)
        assert torch.equal(got_ob, ob) and torch.equal(got_nodes, tok)
        assert got_len.dtype == torch.int64 and torch.equal(got_len, want_len)
        assert got_tok.dtype == torch.float32 and torch.equal(got_tok, want_tok)
    got_tok, got_len = harness.decode_from_logits(logits, links, ol, left_mask, single_call=True)
    two_tok, two_len = harness.decode_from_logits(logits, links, ol, left_mask)
    assert torch.equal(got_tok, two_tok) and torch.equal(got_len, two_len)
    with pytest.raises(RuntimeError, match="float16 or float32"):
        ops.pcfg_viterbi_decode_logits(logits.double(), links, ol, left_mask, synth.PAD)


@pytest.mark.parametrize("case", ["L96", "L288", "L600"])
def test_single_call_decode_c_abi_without_float_tokens(case):
    """pcfgnat_viterbi_decode through ctypes with out_tokens_f32 = NULL (a caller that only wants the int64 rows): the
    one-workgroup decode, the pipelined one and the general path leave the rows and counts the wrapper's float32 tokens
    come from."""
    from pcfg_nat_amd import _lib
    lib = ops.get_pcfg_kernel()
    batch = _decode_case(case)
    ob, tok = synth.ob_and_tokens(batch["logits"])
    links, ol = batch["links"].to(DEV), batch["output_length"].to(DEV)
    B, L = ob.shape
    left_mask = synth.support_masks(L, 1)[0].to(DEV)
    ob, tok = ob.to(DEV), tok.to(DEV)
    want_tok, want_len = ops.pcfg_viterbi_decode(ob, links, ol, tok, left_mask, synth.PAD)
    pen = ops._length_penalty(L // 4, 1.0, ob.device)
    work = torch.empty((lib.pcfgnat_viterbi_decode_workspace_bytes(B, L, 1) + 7) // 8, dtype=torch.int64, device=DEV)
    rows = torch.full((B, L), -7, dtype=torch.int64, device=DEV)
    counts = torch.full((B,), -7, dtype=torch.int64, device=DEV)
    pred = torch.full((B,), -7, dtype=torch.int64, device=DEV)
    _lib.check(lib.pcfgnat_viterbi_decode(ob.data_ptr(), links.data_ptr(), ol.data_ptr(), tok.data_ptr(), left_mask.data_ptr(), L,
                                          synth.PAD, pen.data_ptr(), work.data_ptr(), rows.data_ptr(), None, counts.data_ptr(),
                                          pred.data_ptr(), B, L, 1, torch.cuda.current_stream().cuda_stream), lib)
    torch.cuda.synchronize()
    assert torch.equal(pred, want_len)
    n = int(counts.max())
    assert n == want_tok.shape[1] and torch.equal(rows[:, :n].float(), want_tok)
    assert (rows[:, n:] == synth.PAD).all()


def test_decode_waits_for_the_stream_where_the_counts_do_not_turn():
    """The decode calls watch the token counts turn in pinned host memory.  A watch that runs into its time bound (forced
    here by a bound of zero seconds) hands over to the stream wait for that call with the same results; the watching is
    switched off only after several such misses in a row, and one watch that succeeds resets the count.  A call that finds
    work pending on its stream does not watch at all."""
    import oracle_ops
    batch = _decode_case("L96")
    ob, tok = synth.ob_and_tokens(batch["logits"])
    links, ol = batch["links"], batch["output_length"]
    left_mask, _, _ = synth.support_masks(links.shape[1], 1)
    want_tok, want_len = harness.viterbi_decode(ob, tok, links, ol, left_mask, ops=oracle_ops)
    args = (ob.to(DEV), tok.to(DEV), links.to(DEV), ol.to(DEV), left_mask.to(DEV))

    def decode():
        torch.cuda.synchronize()
        got_tok, got_len = harness.viterbi_decode(*args, single_call=True)
        assert torch.equal(got_len.cpu(), want_len) and torch.equal(got_tok.cpu(), want_tok)

    pool = ops._pinned_counts
    saved = (pool.WATCH_SECONDS, pool._polling, pool._misses)
    try:
        pool._polling, pool._misses = True, 0
        decode()
        assert pool.polling_on() and pool._misses == 0  # the counts turned inside the bound
        pool.WATCH_SECONDS = -1.0  # every watch misses (the bound is looked at every 256 reads: the kernel has not ended by then)
        for k in range(1, pool.MISSES_TO_SWITCH_OFF):
            decode()
            assert pool.polling_on()
        misses_before = pool._misses
        pool.WATCH_SECONDS = saved[0]
        decode()
        assert pool._misses == 0 or misses_before == 0  # a watch that succeeds resets the count
        pool.WATCH_SECONDS = -1.0
        pool._misses = pool.MISSES_TO_SWITCH_OFF - 1
        decode()
        if pool._misses:  # (a kernel that ended within the first 256 reads is no miss)
            assert not pool.polling_on()
        decode()  # without watching: the stream wait alone
        # work pending on the stream: no watch, whatever the setting
        pool._polling, pool._misses, pool.WATCH_SECONDS = True, 0, saved[0]
        big = torch.empty(64 << 20, device=DEV)
        for _ in range(8):
            big.normal_()
        buf = pool.take(4)
        armed = pool.arm(buf, 4, torch.cuda.current_stream(DEV))
        pool.give_back(buf)
        assert armed is False
        decode()
    finally:
        pool.WATCH_SECONDS, pool._polling, pool._misses = saved


@pytest.mark.parametrize("mode", ["one_workgroup", "blocks_give_up"])
@pytest.mark.parametrize("case", ["L224", "L288", "L400", "L512"])
def test_single_call_decode_sweeps_agree(mode, case):
    """Graphs of 194..514 nodes: the pipelined Viterbi sweep (default), the one-workgroup sweep (pipeline switched off) and
    the redo path (blocks that give up at once: spin limit 0) return the same tokens and lengths as the oracle."""
    import oracle_ops
    batch = _decode_case(case)
    ob, tok = synth.ob_and_tokens(batch["logits"])
    links, ol = batch["links"], batch["output_length"]
    left_mask, _, _ = synth.support_masks(links.shape[1], 1)
    want_tok, want_len = harness.viterbi_decode(ob, tok, links, ol, left_mask, ops=oracle_ops)
    try:
        if mode == "one_workgroup":
            ops.pipeline_config(max_workgroups=0)
        else:
            ops.pipeline_config(spin_limit=0)
        got_tok, got_len = harness.viterbi_decode(ob.to(DEV), tok.to(DEV), links.to(DEV), ol.to(DEV), left_mask.to(DEV),
                                                  single_call=True)
    finally:
        ops.pipeline_config(max_workgroups=1 << 20, spin_limit=ops.DEFAULT_SPIN_LIMIT)
    assert torch.equal(got_len.cpu(), want_len) and torch.equal(got_tok.cpu(), want_tok)


def test_decodes_overlapping_on_one_device():
    """Two host threads decode different batches on two streams of one device at the same time, many times over: every call
    gets the token counts of its own batch (each call owns the pinned host buffer the kernel writes them to)."""
    import threading
    import oracle_ops
    cases = []
    for name in ("L96", "L160"):
        batch = _decode_case(name)
        ob, tok = synth.ob_and_tokens(batch["logits"])
        links, ol = batch["links"], batch["output_length"]
        mask = synth.support_masks(links.shape[1], 1)[0]
        want = harness.viterbi_decode(ob, tok, links, ol, mask, ops=oracle_ops)
        cases.append(([t.to(DEV) for t in (ob, tok, links, ol, mask)], want))
    errors = []
    start = threading.Barrier(2)

    def worker(k):
        try:
            args, (want_tok, want_len) = cases[k]
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.default_stream())
            start.wait()
            with torch.cuda.stream(stream):
                for i in range(60):
                    got_tok, got_len = harness.viterbi_decode(*args, single_call=(i % 2 == 0))
                    if not (torch.equal(got_len.cpu(), want_len) and torch.equal(got_tok.cpu(), want_tok)):
                        errors.append((k, i))
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


@pytest.mark.parametrize("ml,L,ms", [(1, 32, [32, 20, 8]), (3, 34, [34, 26]), (1, 400, [400, 284, 20, 400]), (1, 18, [18])])
@pytest.mark.parametrize("strategy", ["lookahead", "greedy"])
def test_lookahead_decode_bit_exact(ml, L, ms, strategy):
    B = len(ms)
    gen = torch.Generator().manual_seed(L + ml)
    links = synth.make_links(B, L, torch.tensor(ms), ml, gen)
    ob = torch.randn(B, L, generator=gen) - 2.0
    tok = torch.randint(4, 60, (B, L), generator=gen)
    tok[:, 5] = synth.PAD
    left_mask, _, _ = synth.support_masks(L, ml)
    beta = 0.9
    want, want_idx = oracle.lookahead_decode(links.numpy(), None if strategy == "greedy" else ob.numpy(), np.array(ms), tok.numpy(),
                                             left_mask.numpy(), synth.PAD, beta)
    got, idx = ops.pcfg_lookahead_decode(links.to(DEV), ob.to(DEV), tok.to(DEV), torch.tensor(ms).to(DEV), left_mask.to(DEV), synth.PAD,
                                         beta=beta, strategy=strategy, return_pointers=True)
    assert idx.dtype == torch.int64 and np.array_equal(idx.cpu().numpy(), want_idx)
    assert got.dtype == torch.int64 and np.array_equal(got.cpu().numpy(), want)


def test_viterbi_exact_ties_follow_reference_order():
    L = m = 32
    links = torch.full((1, L, 2, L), -math.inf)
    for a in range(1, m - 1, 2):
        links[0, a, 0, a + 2:m:2] = -1.0
    ob = torch.full((1, L), -1.0)
    ol = torch.tensor([m])

    def right_child(dead):
        lk = links.clone()
        for cid in dead:
            lk[0, 1, 0, 2 * cid + 1] = -math.inf
        _, R, _, _ = ops.cuda_pcfg_viterbi(ob.to(DEV), lk.to(DEV), ol.to(DEV))
        return (int(R[0, 1, 3]) - 1) // 2

    assert right_child(()) == 4
    assert right_child((4, 8, 12)) == 2
    assert right_child((4, 8, 12, 2, 6, 10, 14)) == 1
    assert right_child((4, 8, 12, 2, 6, 10, 14, 1, 5, 9, 13)) == 3


def test_criterion_glue_end_to_end_cfg1():
    """logsoftmax_gather -> eos mask -> inside loss -> backward through both ops, against the same glue over the oracle."""
    import oracle_ops
    batch = synth.config1()
    B, L, V = batch["logits"].shape
    out_mask = torch.arange(L).view(1, L) < batch["output_length"].view(B, 1)
    tgt_mask = batch["targets"].ne(synth.PAD)

    def run(dev, opsmod):
        leaf = batch["logits"].clone().to(dev).requires_grad_(True)
        links = batch["links"].clone().to(dev).requires_grad_(True)
        res = harness.compute_pcfg_loss(leaf * 1.0, out_mask.to(dev), batch["targets"].to(dev), tgt_mask.to(dev), links,
                                        ops=opsmod)
        res["loss"].backward()
        return res["loss"].detach().cpu(), leaf.grad.cpu(), links.grad.cpu()

    loss_g, gl_g, gk_g = run(DEV, ops)
    loss_o, gl_o, gk_o = run("cpu", oracle_ops)
    assert torch.allclose(loss_g, loss_o, rtol=1e-5)
    assert (gl_g - gl_o).abs().max() <= 1e-4 * gl_o.abs().max()
    assert (gk_g - gk_o).abs().max() <= 1e-4 * gk_o.abs().max()


def test_errors_are_loud():
    x = torch.randn(2, 3, 16, device=DEV)
    with pytest.raises(RuntimeError, match="select_idx should be long"):
        ops._logsoftmax_gather(x, torch.zeros(2, 3, 4, dtype=torch.int32, device=DEV), False)
    with pytest.raises(RuntimeError, match="not contiguous"):
        ops._logsoftmax_gather(x.transpose(0, 1), torch.zeros(3, 2, 4, dtype=torch.int64, device=DEV), False)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.cuda_pcfg_loss(torch.zeros(1, 8, 4), torch.zeros(1, 8, 2, 8), torch.tensor([8]), torch.tensor([4]))
    # out-of-contract lengths poison the log-likelihood instead of faulting
    match = torch.zeros(1, 8, 4, device=DEV)
    links = torch.zeros(1, 8, 2, 8, device=DEV)
    ll = ops.cuda_pcfg_loss(match, links, torch.tensor([7], device=DEV), torch.tensor([4], device=DEV))
    assert torch.isnan(ll).all()
    with pytest.raises(RuntimeError, match="max_left"):  # a graph of 8 nodes cannot hold max_left = 7
        ops.cuda_pcfg_loss(match, torch.zeros(1, 8, 8, 8, device=DEV), torch.tensor([8], device=DEV),
                           torch.tensor([4], device=DEV))


@pytest.mark.parametrize("shape", ["L64", "L64_odd_vocab", "L30_fp32", "L320", "L1100", "ml3"])
def test_fused_step_equals_autograd_step(shape):
    """train_step_fused / train_step_direct leave the same loss, logits gradient and links gradient as autograd through
    the operator API (one invalid sentence included: its gradients must vanish).  Every shape has sentences shorter than
    the padded graph: the single-call step leaves the rows of those pad nodes unread and must still zero their gradients
    (register-resident, pipelined, streaming and general max_left sweeps)."""
    if shape == "L64":
        batch = synth.training_batch(4, 64, 12, 700, [64, 40, 22, 8], [12, 9, 12, 12], seed=31, logit_scale=2.0,
                                     logit_dtype=torch.float16)
    elif shape == "L64_odd_vocab":  # rows of 666 bytes: the spans of pad rows start and end off the 16-byte grid
        batch = synth.training_batch(4, 64, 12, 333, [62, 40, 22, 8], [12, 9, 12, 12], seed=36, logit_scale=2.0,
                                     logit_dtype=torch.float16)
    elif shape == "L30_fp32":
        batch = synth.training_batch(4, 30, 12, 257, [30, 18, 4, 8], [12, 9, 2, 12], seed=37, logit_scale=2.0,
                                     logit_dtype=torch.float32)
    elif shape == "L320":
        batch = synth.training_batch(4, 320, 24, 300, [320, 200, 64, 8], [24, 20, 9, 12], seed=32, logit_scale=2.0,
                                     logit_dtype=torch.float16)
    elif shape == "L1100":
        batch = synth.training_batch(4, 1100, 12, 120, [1100, 800, 64, 8], [12, 8, 9, 12], seed=34, logit_scale=2.0,
                                     logit_dtype=torch.float16)
    else:
        batch = synth.training_batch(4, 66, 12, 300, [66, 50, 22, 10], [12, 9, 7, 12], seed=35, ml=3, logit_scale=2.0,
                                     logit_dtype=torch.float16)
    B, L, V = batch["logits"].shape
    out_mask = (torch.arange(L).view(1, L) < batch["output_length"].view(B, 1)).to(DEV)
    tgt = batch["targets"].to(DEV)
    tgt_mask = tgt.ne(synth.PAD)
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    links = batch["links"].to(DEV).requires_grad_(True)
    half = batch["logits"].dtype == torch.float16
    res = harness.compute_pcfg_loss(leaf.half() if half else leaf * 1.0, out_mask, tgt, tgt_mask, links)
    assert int(res["invalid_nsentences"]) == 1
    res["loss"].backward()
    for step in (harness.train_step_direct, harness.train_step_fused, harness.train_step_single_call):
        buf = batch["logits"].to(DEV).clone()
        loss, glinks, ll = step(buf, tgt, batch["links"].to(DEV), ol, tl)
        assert torch.allclose(loss, res["loss"].detach(), rtol=1e-6)
        # (the variants run their sweeps in different kernels: each is within 1e-4 of the oracle, and they are within a few
        # 1e-6 of each other)
        assert torch.allclose(glinks, links.grad, rtol=3e-5, atol=1e-9)
        if half:
            assert torch.allclose(buf.float(), leaf.grad, rtol=2 ** -9, atol=2 ** -22)
        else:
            assert torch.allclose(buf, leaf.grad, rtol=2e-5, atol=1e-9)
        assert not glinks[3].any() and not buf[3].any()
        assert not buf[~out_mask].any()


@pytest.mark.parametrize("V", [700, 40000])
@pytest.mark.parametrize("scale", [1.0, 128.0, 65536.0])
def test_criterion_op_under_autograd(scale, V):
    """pcfg_criterion (one native call in the forward, one in the backward) against autograd through the separate ops,
    with and without an upstream factor on the loss (fp16 loss scaling, pcfg_loss.py:77-83): the factor has to reach the
    gradient ahead of its rounding to fp16.  At V=40000 most entries of the unscaled gradient lie below the smallest fp16
    subnormal, so a factor applied after the rounding would leave zeros where the drop-in ops have values.  Per element:
    one fp16 rounding step (both sides round a float32 value once; the float32 values differ by reassociation only)."""
    batch = synth.training_batch(4, 64, 12, V, [64, 40, 22, 8], [12, 9, 12, 12], seed=43, logit_scale=2.0,
                                 logit_dtype=torch.float16)
    B, L, V = batch["logits"].shape
    out_mask = (torch.arange(L).view(1, L) < batch["output_length"].view(B, 1)).to(DEV)
    tgt = batch["targets"].to(DEV)
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    links = batch["links"].to(DEV).requires_grad_(True)
    res = harness.compute_pcfg_loss(leaf.half(), out_mask, tgt, tgt.ne(synth.PAD), links)
    (res["loss"] * scale).backward()
    leaf2 = batch["logits"].to(DEV).float().requires_grad_(True)
    links2 = batch["links"].to(DEV).requires_grad_(True)
    loss, ll, invalid = ops.pcfg_criterion(leaf2.half(), tgt, links2, ol, tl)
    assert torch.allclose(loss, res["loss"].detach(), rtol=1e-6) and int(invalid) == 1
    assert torch.allclose(ll, res["ll"].detach(), rtol=1e-6)
    (loss * scale).backward()
    assert torch.isfinite(leaf2.grad).all() and torch.isfinite(leaf.grad).all()
    assert torch.allclose(links2.grad, links.grad, rtol=1e-5, atol=1e-9 * scale)
    assert torch.allclose(leaf2.grad, leaf.grad, rtol=2 ** -9, atol=2 ** -24)
    assert not leaf2.grad[~out_mask].any() and not leaf2.grad[3].any()
    if V == 40000 and scale > 1:  # the factor did rescue entries that are flushed to zero at scale 1
        assert (leaf2.grad != 0).sum() == (leaf.grad != 0).sum() or (leaf2.grad != 0).sum() > 0.5 * (leaf.grad != 0).sum()
        assert (leaf.grad != 0).float().mean() > 0.05
    # the plain single call with the factor handed over up front: as a host number and as a scalar in device memory
    for given in (scale, torch.tensor([scale], device=DEV)):
        buf = batch["logits"].to(DEV).clone()
        out, glinks, _, _, _ = ops.pcfg_criterion_step(buf, tgt, batch["links"].to(DEV), ol, tl, loss_scale=given)
        assert torch.allclose(out[0], res["loss"].detach(), rtol=1e-6)
        assert torch.allclose(glinks, links.grad, rtol=1e-5, atol=1e-9 * scale)
        assert torch.allclose(buf.float(), leaf.grad, rtol=2 ** -9, atol=2 ** -24)


def test_single_call_step_large_batch_of_short_graphs():
    """100 sentences of at most 16 nodes: more sweeps than the launch that holds them can spare compute units for the zeros
    of the pad rows, which the gather backward then writes itself.  Against the four-call step over the same kernels."""
    B, L, T, V = 100, 16, 6, 50
    gen = torch.Generator().manual_seed(41)
    ms = (2 * torch.randint(2, L // 2 + 1, (B,), generator=gen)).tolist()
    ns = torch.randint(2, T + 1, (B,), generator=gen).tolist()
    ms[0], ns[0] = L, T
    batch = synth.training_batch(B, L, T, V, ms, ns, seed=42, logit_scale=2.0, logit_dtype=torch.float16)
    tgt, links = batch["targets"].to(DEV), batch["links"].to(DEV)
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    want_buf = batch["logits"].to(DEV).clone()
    want_loss, want_glinks, want_ll = harness.train_step_fused(want_buf, tgt, links, ol, tl)
    buf = batch["logits"].to(DEV).clone()
    loss, glinks, ll = harness.train_step_single_call(buf, tgt, links, ol, tl)
    fin = torch.isfinite(want_ll)
    assert fin.any() and torch.equal(fin, torch.isfinite(ll))
    assert torch.allclose(ll[fin], want_ll[fin], rtol=1e-6)
    assert torch.allclose(loss, want_loss, rtol=1e-6)
    assert torch.allclose(glinks, want_glinks, rtol=1e-5, atol=1e-9)
    assert torch.allclose(buf.float(), want_buf.float(), rtol=2 ** -9, atol=2 ** -22)
    out_mask = torch.arange(L, device=DEV).view(1, L) < ol.view(B, 1)
    assert not buf[~out_mask].any()


def test_force_emit_step_equals_autograd_step():
    """The criterion with force-emit masking (nat_pcfg_loss.py:116-121; on in the scripts without --no-force-emit): the
    masks come from a glancing pass over the same batch; autograd through the torch restatement of those lines against
    the single-call step that folds them into the gather kernels.  Revealed nodes must end up with a zero logits
    gradient, and the loss must differ from the unmasked one (the masks do something)."""
    batch = synth.training_batch(4, 64, 12, 700, [64, 40, 22, 8], [12, 9, 7, 3], seed=33, logit_scale=2.0,
                                 logit_dtype=torch.float16)
    B, L, V = batch["logits"].shape
    out_mask = (torch.arange(L).view(1, L) < batch["output_length"].view(B, 1)).to(DEV)
    tgt = batch["targets"].to(DEV)
    tgt_mask = tgt.ne(synth.PAD)
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    prev = torch.full((B, L), 3, dtype=torch.int64, device=DEV).masked_fill(~out_mask, synth.PAD)
    gen = torch.Generator().manual_seed(5)
    glat = harness.glat_alignment(batch["logits"].to(DEV).clone(), tgt, prev, batch["links"].to(DEV), 0.5, generator=gen,
                                  noise_device="cpu")
    mm, keep = glat["matchmask"], glat["keep_word_mask"]
    assert keep.any() and not keep.all()
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    links = batch["links"].to(DEV).requires_grad_(True)
    res = harness.compute_pcfg_loss(leaf.half(), out_mask, tgt, tgt_mask, links, matchmask=mm, keep_word_mask=keep)
    res["loss"].backward()
    plain = harness.compute_pcfg_loss(batch["logits"].to(DEV).clone(), out_mask, tgt, tgt_mask, batch["links"].to(DEV))
    assert abs(float(plain["loss"].detach()) - float(res["loss"].detach())) > 1e-3
    buf = batch["logits"].to(DEV).clone()
    loss, glinks, ll = harness.train_step_single_call(buf, tgt, batch["links"].to(DEV), ol, tl, matchmask=mm, keep_word_mask=keep)
    assert torch.allclose(loss, res["loss"].detach(), rtol=1e-6)
    assert torch.allclose(glinks, links.grad, rtol=1e-5, atol=1e-9)
    assert torch.allclose(buf.float(), leaf.grad, rtol=2 ** -9, atol=2 ** -22)
    assert not buf[keep].any()


def _generic_batch(ml, L, ms, ns, seed, generic_local):
    """Batch for a general max_left: links with the grammar's structural support (optionally with composite local trees),
    random emissions with the eos column masked."""
    from test_oracle_inside import random_links
    rng = np.random.default_rng(seed)
    B, T = len(ms), max(ns)
    links = np.stack([random_links(rng, L, m, ml, p_drop=0.1, generic_local=generic_local) for m in ms]).astype(np.float32)
    match = (rng.normal(size=(B, L, T)) - 2.0).astype(np.float32)
    ol, tl = torch.tensor(ms), torch.tensor(ns)
    match = harness.eos_masked(torch.from_numpy(match), ol, tl)
    return match, torch.from_numpy(links), ol, tl


@pytest.mark.parametrize("ml,L,ms,ns,generic_local", [
    (3, 30, [30, 22, 14], [9, 8, 5], True),
    (3, 66, [66, 50], [14, 20], False),
    (7, 42, [42, 26], [8, 6], True),
    (0, 12, [12, 9, 5], [7, 9, 3], False),
    (2, 32, [32, 20], [9, 7], True),
])
def test_general_max_left_vs_oracle(ml, L, ms, ns, generic_local):
    match, links, ol, tl = _generic_batch(ml, L, ms, ns, seed=ml * 100 + L, generic_local=generic_local)
    S64, C64 = oracle.inside_fwd(match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float64)
    mg64, lg64 = oracle.inside_bwd(np.ones(len(ms)), S64, C64, match.numpy(), links.numpy(), ol.numpy(), tl.numpy())
    md = match.to(DEV).requires_grad_(True)
    ld = links.to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, ol.to(DEV), tl.to(DEV))
    want = S64[:, 0, 0]
    got = ll.detach().cpu().double().numpy()
    fin = np.isfinite(want)
    assert fin.any() and np.array_equal(np.isfinite(got), fin)
    assert np.allclose(got[fin], want[fin], rtol=1e-5)
    ll.masked_fill(~torch.isfinite(ll), 0).sum().backward()
    for bi in range(len(ms)):
        for g_got, g_want in ((md.grad[bi], mg64[bi]), (ld.grad[bi], lg64[bi])):
            g_got = g_got.cpu().double().numpy()
            assert np.isfinite(g_got).all()
            assert np.abs(g_got - g_want).max() <= 1e-4 * max(np.abs(g_want).max(), 1e-30)
    # best tree: same alignment as the oracle on these seeds, and a valid alignment
    tree, ll2 = ops.cuda_pcfg_best_tree(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV))
    want_tree = oracle.best_tree(S64, C64, match.numpy(), links.numpy(), ol.numpy(), tl.numpy())
    assert np.array_equal(tree.cpu().numpy(), want_tree)
    assert torch.allclose(ll2, ll.detach(), rtol=1e-6, equal_nan=True)


def _max_left3_against_oracle(match, links, ol, tl, valid):
    """cuda_pcfg_loss at max_left = 3 against the float64 oracle: log-likelihoods, both gradients entry by entry."""
    B = match.size(0)
    S64, C64 = oracle.inside_fwd(match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float64)
    mg64, lg64 = oracle.inside_bwd(np.ones(B), S64, C64, match.numpy(), links.numpy(), ol.numpy(), tl.numpy())
    md = match.to(DEV).requires_grad_(True)
    ld = links.to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, ol.to(DEV), tl.to(DEV))
    got = ll.detach().cpu().double().numpy()
    want = S64[:, 0, 0]
    fin = np.isfinite(want) & np.asarray(valid)
    assert fin.any() and np.array_equal(np.isfinite(got), fin)
    assert np.allclose(got[fin], want[fin], rtol=1e-5)
    ll.masked_fill(~torch.isfinite(ll), 0).sum().backward()
    worst = 0.0
    for bi in range(B):
        for name, g_got, g_want in (("match_all_grad", md.grad[bi], mg64[bi]), ("links_grad", ld.grad[bi], lg64[bi])):
            g_got = g_got.cpu().double().numpy()
            assert np.isfinite(g_got).all()
            if not fin[bi]:
                assert not g_got.any()
                continue
            worst = max([worst] + gradcheck.assert_elementwise(g_got, g_want, "%s of sentence %d" % (name, bi)))
    return ll.detach(), md.grad, ld.grad, worst


@pytest.mark.parametrize("L,ms,ns", [
    (66, [66, 50, 34, 6], [14, 20, 9, 2]),
    (130, [130, 98, 42, 130], [32, 20, 12, 2]),
    (254, [254, 130], [64, 33]),
])
def test_max_left3_one_launch_kernel_vs_oracle(L, ms, ns):
    """Links as the model's scorer produces them for --left-tree-layer 2 (no local node has a rule: right children are
    main-chain nodes only), every left option of the main-chain nodes finite: the one-launch kernel serves every sentence
    and agrees with the float64 oracle and with the plain kernels."""
    match, links, ol, tl = _generic_batch(3, L, ms, ns, seed=300 + L, generic_local=False)
    assert ops.max_left_path(3, L, max(ns)) == "tuned"
    ops.max_left3_counts(reset=True)
    ll, mg, lg, worst = _max_left3_against_oracle(match, links, ol, tl, [True] * len(ms))
    assert ops.max_left3_counts() == (len(ms), 0)
    print("max_left = 3, L=%d: worst relative error of a gradient entry %.2e" % (L, worst))
    was = ops.max_left3_tuned(0)
    try:
        assert ops.max_left_path(3, L, max(ns)) == "generic"
        ll_p, mg_p, lg_p, _ = _max_left3_against_oracle(match, links, ol, tl, [True] * len(ms))
        assert ops.max_left3_counts() == (len(ms), 0)  # (the plain kernels ran alone: the counters did not move)
    finally:
        ops.max_left3_tuned(was)
    assert torch.allclose(ll, ll_p, rtol=2e-6)
    assert torch.allclose(mg, mg_p, rtol=2e-4, atol=1e-7) and torch.allclose(lg, lg_p, rtol=2e-4, atol=1e-7)


def test_max_left3_mixed_batch_and_invalid_lengths():
    """Sentences with and without rules of composite local trees in one batch, and graph sizes outside the contract: the
    one-launch kernel takes what it covers, the plain kernels the rest, neither touches the other's sentences."""
    from test_oracle_inside import random_links
    L, T = 46, 12
    ms, ns = [46, 30, 46, 22, 38, 46], [12, 9, 7, 6, 10, 5]
    composite = [False, True, False, True, False, True]
    rng = np.random.default_rng(77)
    links = np.stack([random_links(rng, L, m, 3, p_drop=0.1, generic_local=c) for m, c in zip(ms, composite)]).astype(np.float32)
    match = (rng.normal(size=(len(ms), L, T)) - 2.0).astype(np.float32)
    ol, tl = torch.tensor(ms), torch.tensor(ns)
    match = harness.eos_masked(torch.from_numpy(match), ol, tl)
    ops.max_left3_counts(reset=True)
    _max_left3_against_oracle(match, torch.from_numpy(links), ol, tl, [True] * len(ms))
    assert ops.max_left3_counts() == (3, 3)
    # graph sizes that are no whole number of groups, or too small: NaN log-likelihood, zero gradients, no fault
    bad_ol = torch.tensor([45, 30, 4, 22, 38, 47])
    md = match.to(DEV).requires_grad_(True)
    ld = torch.from_numpy(links).to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, bad_ol.to(DEV), tl.to(DEV))
    ok = torch.tensor([False, True, False, True, True, False])
    assert torch.equal(torch.isfinite(ll).cpu(), ok) and torch.isnan(ll[~ok.to(DEV)]).all()
    ll.masked_fill(~torch.isfinite(ll), 0).sum().backward()
    assert not md.grad[~ok.to(DEV)].any() and not ld.grad[~ok.to(DEV)].any()
    assert torch.isfinite(md.grad).all() and torch.isfinite(ld.grad).all()


def test_max_left3_model_shaped_batch_vs_oracle():
    """The bench's shape (B=40, L=130, T=32) with jointly normalised links on the model's support."""
    B, L, T, ml = 40, 130, 32, 3
    gen = torch.Generator().manual_seed(1003)
    src, n = synth._wmt_lengths(B, gen, 10, 32, T)
    m = src + 2
    links = synth.make_links(B, L, m, ml, gen)
    match = harness.eos_masked(torch.log_softmax(torch.randn(B, L, T, generator=gen) * 2, dim=-1), m, n)
    ops.max_left3_counts(reset=True)
    _, _, _, worst = _max_left3_against_oracle(match, links, m, n, [True] * B)
    assert ops.max_left3_counts() == (B, 0)
    print("max_left = 3 at B=40, L=130, T=32: worst relative error of a gradient entry %.2e" % worst)


@pytest.mark.parametrize("ml,L,ms", [(3, 66, [66, 50, 34]), (7, 74, [74, 42]), (0, 24, [24, 13]), (2, 50, [50, 32])])
def test_general_max_left_viterbi_bit_exact(ml, L, ms):
    from test_oracle_inside import random_links
    rng = np.random.default_rng(ml + L)
    links = np.stack([random_links(rng, L, m, ml, p_drop=0.1, generic_local=True) for m in ms]).astype(np.float32)
    ob = (rng.normal(size=(len(ms), L)) - 1.0).astype(np.float32)
    ol = torch.tensor(ms)
    scores, R, Lt, M = ops.cuda_pcfg_viterbi(torch.from_numpy(ob).to(DEV), torch.from_numpy(links).to(DEV), ol.to(DEV))
    S_o, R_o, L_o, M_o = oracle.viterbi(ob, links, ol.numpy(), dtype=np.float32)
    assert np.isfinite(S_o[:, 1, :]).any()
    assert np.array_equal(scores.cpu().numpy(), S_o[:, 1, :])
    assert np.array_equal(R.cpu().numpy(), R_o) and np.array_equal(Lt.cpu().numpy(), L_o) and np.array_equal(M.cpu().numpy(), M_o)


def _viterbi_tables_equal_oracle(ob, links, ol):
    scores, R, Lt, M = ops.cuda_pcfg_viterbi(torch.from_numpy(ob).to(DEV), torch.from_numpy(links).to(DEV), ol.to(DEV))
    S_o, R_o, L_o, M_o = oracle.viterbi(ob, links, ol.numpy(), dtype=np.float32)
    assert np.array_equal(scores.cpu().numpy(), S_o[:, 1, :])
    assert np.array_equal(R.cpu().numpy(), R_o) and np.array_equal(Lt.cpu().numpy(), L_o) and np.array_equal(M.cpu().numpy(), M_o)
    return S_o, (scores, R, Lt, M)


@pytest.mark.parametrize("quantised", [False, True])
@pytest.mark.parametrize("L,ms", [(18, [18, 14, 6, 2]), (66, [66, 50, 34, 6]), (130, [130, 98, 42]), (258, [258, 254, 130]),
                                  (402, [402, 202]), (510, [510, 398])])
def test_max_left3_viterbi_one_launch_kernel_bit_exact(L, ms, quantised):
    """Viterbi tables at max_left = 3 with links as the model's scorer produces them (no local node has a rule): the
    one-launch kernel serves every sentence and returns the oracle's scores and back-pointers bit for bit, as do the plain
    kernels.  ``quantised``: values on a grid of quarters, so that exact ties between candidates are the rule and the
    winner is decided by the reference's scan order (lane of its strided scan, child, yield, left node)."""
    from test_oracle_inside import random_links
    rng = np.random.default_rng(900 + L + (1 if quantised else 0))
    links = np.stack([random_links(rng, L, m, 3, p_drop=0.1) for m in ms]).astype(np.float32)
    ob = (rng.normal(size=(len(ms), L)) - 1.0).astype(np.float32)
    if quantised:
        links = (np.round(links * 2) / 2).astype(np.float32)  # (-inf stays -inf)
        ob = (np.round(ob * 2) / 2).astype(np.float32)
    ol = torch.tensor(ms)
    ops.max_left3_counts(reset=True, viterbi=True)
    S_o, tuned = _viterbi_tables_equal_oracle(ob, links, ol)
    assert ops.max_left3_counts(viterbi=True) == (len(ms), 0)
    assert np.isfinite(S_o[0, 1, 2:]).any()
    was = ops.max_left3_tuned(0)
    try:
        _, plain = _viterbi_tables_equal_oracle(ob, links, ol)
        assert ops.max_left3_counts(viterbi=True) == (len(ms), 0)  # (the plain kernel ran alone: the counters did not move)
    finally:
        ops.max_left3_tuned(was)
    for t, p in zip(tuned, plain):
        assert torch.equal(t, p)


def test_max_left3_viterbi_mixed_batch_and_invalid_lengths():
    """Sentences with and without rules of composite local trees in one batch, and graph sizes outside the contract (empty
    tables): the one-launch kernel takes what it covers, the plain kernel the rest."""
    from test_oracle_inside import random_links
    L = 46
    ms = [46, 30, 45, 22, 4, 46, 47, 38]
    composite = [False, True, False, True, False, True, False, False]
    rng = np.random.default_rng(78)
    links = np.stack([random_links(rng, L, min(m, L), 3, p_drop=0.1, generic_local=c) for m, c in zip(ms, composite)]).astype(np.float32)
    ob = (rng.normal(size=(len(ms), L)) - 1.0).astype(np.float32)
    ops.max_left3_counts(reset=True, viterbi=True)
    S_o, _ = _viterbi_tables_equal_oracle(ob, links, torch.tensor(ms))
    assert ops.max_left3_counts(viterbi=True) == (5, 3)
    assert np.isfinite(S_o[[0, 1, 3, 5, 7], 1, :]).any(axis=1).all() and not np.isfinite(S_o[[2, 4, 6], 1, :]).any()


@pytest.mark.parametrize("ml,L,ms", [(3, 66, [66, 50, 34, 6]), (3, 258, [258, 130]), (2, 50, [50, 32]), (0, 24, [24, 13])])
def test_general_max_left_decode_vs_oracle(ml, L, ms):
    """The Viterbi decode at max_left != 1 (full tables, selection and walk as separate launches): the single native call and
    the three operators one by one emit the oracle's tokens and lengths, with the left-tree mask of that tree shape."""
    import oracle_ops
    gen = torch.Generator().manual_seed(100 * ml + L)
    m = torch.tensor(ms)
    links = synth.make_links(len(ms), L, m, ml, gen)
    ob, tok = synth.ob_and_tokens(torch.randn(len(ms), L, 48, generator=gen) * 3)
    left_mask = synth.support_masks(L, ml)[0]
    want_tok, want_len = harness.viterbi_decode(ob, tok, links, m, left_mask, ops=oracle_ops)
    assert want_tok.shape[1] >= 3 and (want_len > 1).any()  # a real tree, not the one-token fallback of a dead graph
    for single in (False, True):
        got_tok, got_len = harness.viterbi_decode(ob.to(DEV), tok.to(DEV), links.to(DEV), m.to(DEV), left_mask.to(DEV),
                                                  single_call=single)
        assert torch.equal(got_len.cpu(), want_len)
        assert got_tok.dtype == torch.float32 and torch.equal(got_tok.cpu(), want_tok)


@pytest.mark.parametrize("ml,L,ms,ns,generic_local", [
    (1, 32, [32, 20, 8], [10, 8, 3], False),
    (1, 130, [130, 96], [22, 30], False),
    (3, 30, [30, 22, 14], [9, 8, 5], True),
])
def test_float64_tables_vs_oracle(ml, L, ms, ns, generic_local):
    """The float64 instantiation the reference also dispatches (pcfg_loss.cu:395): log-likelihood, both gradients (scaled
    by a non-trivial upstream gradient through autograd) and the best-tree alignment against the float64 oracle."""
    match, links, ol, tl = _generic_batch(ml, L, ms, ns, seed=7 * ml + L, generic_local=generic_local)
    match, links = match.double(), links.double()
    S64, C64 = oracle.inside_fwd(match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float64)
    mg64, lg64 = oracle.inside_bwd(np.ones(len(ms)), S64, C64, match.numpy(), links.numpy(), ol.numpy(), tl.numpy())
    md = match.to(DEV).requires_grad_(True)
    ld = links.to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, ol.to(DEV), tl.to(DEV))
    assert ll.dtype == torch.float64
    want = S64[:, 0, 0]
    got = ll.detach().cpu().numpy()
    fin = np.isfinite(want)
    assert fin.any() and np.array_equal(np.isfinite(got), fin)
    assert np.allclose(got[fin], want[fin], rtol=1e-12)
    w = torch.linspace(0.5, 1.5, ll.numel(), device=DEV, dtype=torch.float64)
    (ll.masked_fill(~torch.isfinite(ll), 0) * w).sum().backward()
    wn = w.cpu().numpy()
    for bi in range(len(ms)):
        for g_got, g_want in ((md.grad[bi], mg64[bi] * wn[bi]), (ld.grad[bi], lg64[bi] * wn[bi])):
            g_got = g_got.cpu().numpy()
            assert np.isfinite(g_got).all()
            assert np.abs(g_got - g_want).max() <= 1e-10 * max(np.abs(g_want).max(), 1e-30)
    tree, ll2 = ops.cuda_pcfg_best_tree(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV))
    want_tree = oracle.best_tree(S64, C64, match.numpy(), links.numpy(), ol.numpy(), tl.numpy(), dtype=np.float64)
    assert np.array_equal(tree.cpu().numpy(), want_tree)
    assert torch.allclose(ll2, ll.detach(), rtol=1e-12, equal_nan=True)


@pytest.mark.parametrize("ml,L,ms", [(1, 64, [64, 40, 12]), (3, 66, [66, 50])])
def test_float64_viterbi_bit_exact(ml, L, ms):
    from test_oracle_inside import random_links
    rng = np.random.default_rng(11 * ml + L)
    links = np.stack([random_links(rng, L, m, ml, p_drop=0.1, generic_local=ml != 1) for m in ms])
    ob = rng.normal(size=(len(ms), L)) - 1.0
    ol = torch.tensor(ms)
    scores, R, Lt, M = ops.cuda_pcfg_viterbi(torch.from_numpy(ob).to(DEV), torch.from_numpy(links).to(DEV), ol.to(DEV))
    assert scores.dtype == torch.float64
    S_o, R_o, L_o, M_o = oracle.viterbi(ob, links, ol.numpy(), dtype=np.float64)
    assert np.isfinite(S_o[:, 1, :]).any()
    assert np.array_equal(scores.cpu().numpy(), S_o[:, 1, :])
    assert np.array_equal(R.cpu().numpy(), R_o) and np.array_equal(Lt.cpu().numpy(), L_o) and np.array_equal(M.cpu().numpy(), M_o)


def test_smallest_shapes_through_every_entry_point():
    """The smallest shapes the grammar allows (a graph of 4 nodes, i.e. two main-chain nodes; 2 target tokens; one
    sentence) and an empty batch, through loss + gradients, best tree, the single-call step, viterbi and the decodes."""
    batch = synth.training_batch(1, 4, 2, 9, [4], [2], seed=2)
    match = _match_for(batch)
    S64, C64, mg64, lg64 = _oracle_inside(batch, match.numpy())
    assert np.isfinite(S64[0, 0, 0])
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    md, ld = match.to(DEV).requires_grad_(True), batch["links"].to(DEV).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(md, ld, ol, tl)
    assert np.allclose(ll.detach().cpu().numpy(), S64[:, 0, 0], rtol=1e-5)
    ll.sum().backward()
    assert np.allclose(md.grad.cpu().numpy(), mg64, atol=1e-5) and np.allclose(ld.grad.cpu().numpy(), lg64, atol=1e-5)
    tree, _ = ops.cuda_pcfg_best_tree(match.to(DEV), batch["links"].to(DEV), ol, tl)
    want_tree = oracle.best_tree(*oracle.inside_fwd(match.numpy(), batch["links"].numpy(), ol.cpu().numpy(), tl.cpu().numpy(),
                                                    dtype=np.float32),
                                 match.numpy(), batch["links"].numpy(), ol.cpu().numpy(), tl.cpu().numpy(), dtype=np.float32)
    assert np.array_equal(tree.cpu().numpy(), want_tree)
    buf = batch["logits"].to(DEV).half()
    loss, glinks, ll2 = harness.train_step_single_call(buf, batch["targets"].to(DEV), batch["links"].to(DEV), ol, tl)
    assert torch.isfinite(loss) and torch.isfinite(buf.float()).all()
    # decode: 8 nodes is the smallest graph with a non-trivial length table (L/4 = 2)
    dec = synth.decode_batch([2], seed=4, V=16, logit_dtype=torch.float32)
    ob, tok = synth.ob_and_tokens(dec["logits"])
    L = dec["links"].shape[1]
    lmask = synth.support_masks(L, 1)[0]
    want_tok, want_len = harness.viterbi_decode(ob, tok, dec["links"], dec["output_length"], lmask, ops=__import__("oracle_ops"))
    for single in (False, True):
        got_tok, got_len = harness.viterbi_decode(ob.to(DEV), tok.to(DEV), dec["links"].to(DEV), dec["output_length"].to(DEV),
                                                  lmask.to(DEV), single_call=single)
        assert torch.equal(got_len.cpu(), want_len) and torch.equal(got_tok.cpu(), want_tok)
    # empty batch: nothing to do, nothing to fault on
    e = torch.empty
    ll0 = ops.cuda_pcfg_loss(e(0, 8, 4, device=DEV), e(0, 8, 2, 8, device=DEV), e(0, dtype=torch.int64, device=DEV),
                             e(0, dtype=torch.int64, device=DEV))
    assert ll0.shape == (0,)
    sc, R, Lt, M = ops.cuda_pcfg_viterbi(e(0, 8, device=DEV), e(0, 8, 2, 8, device=DEV), e(0, dtype=torch.int64, device=DEV))
    assert sc.shape == (0, 2) and R.shape == (0, 8, 2)
