"""The BASELINE configurations at their full sizes on the GPU: checked against torch's library routines on the device,
against the CPU oracle on every sentence (float64 tables), and through size-independent properties (posterior mass per
target token, rule mass = emission mass, softmax rows summing to one, gradients of the gathered logits summing to zero).
The smallest arg-max margins the oracle meets on the way (best tree, Viterbi) are printed per configuration.
"""
import numpy as np
import pytest
import torch

import gradcheck
import oracle_ops
from oracle import oracle
from pcfg_nat_amd import custom_ops as ops
from pcfg_nat_amd import harness, synth

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _check_training_batch(batch, chunk, grad_tol=1e-4):
    B, L, V = batch["logits"].shape
    T = batch["targets"].shape[1]
    ol, tl = batch["output_length"], batch["target_length"]
    logits = batch["logits"].to(DEV)
    targets, links = batch["targets"].to(DEV), batch["links"].to(DEV)
    idx = targets.unsqueeze(1).expand(-1, L, -1)
    want_sel = torch.log_softmax(logits.float(), -1).gather(-1, idx)
    want_sel = harness.eos_masked(want_sel, ol.to(DEV), tl.to(DEV))
    buf = logits.clone()
    out, glinks, ll, match, mgrad = ops.pcfg_criterion_step(buf, targets, links, ol.to(DEV), tl.to(DEV))
    # the step leaves the rows of the pad nodes behind each sentence's graph unread: zeros in `match`, zero gradients
    live = (torch.arange(L).view(1, L) < ol.view(B, 1)).to(DEV)
    fin = torch.isfinite(want_sel) & live.unsqueeze(-1)
    assert torch.equal(torch.isfinite(match) & live.unsqueeze(-1), fin)
    assert torch.allclose(match[fin], want_sel[fin], rtol=2e-5, atol=2e-5)
    assert not match[~live].any() and not buf[~live].any()
    assert torch.isfinite(ll).all() and float(out[1]) == 0
    assert torch.allclose(out[0], -(ll / tl.to(DEV)).mean(), rtol=1e-6)
    # gradient of the loss w.r.t. the logits: every row sums to ~0 (softmax), fp16 storage
    g = buf.float()
    assert torch.isfinite(g).all()
    # (each of the V entries is rounded to fp16, most of them in the subnormal range whose spacing is 2^-24)
    row_sums = g.sum(-1).abs().max().item()
    assert row_sums < V * 2.0 ** -25 + 1e-6
    # every target token is emitted by exactly one node: posterior mass per position = d loss / d ll_b
    coef = (-1.0 / (tl.double() * B))
    mgd = mgrad.double().cpu()
    lg = glinks.double().cpu()
    assert torch.isfinite(lg).all() and torch.isfinite(mgd).all()
    pos = torch.arange(T).view(1, T)
    want_mass = torch.where(pos < tl.view(B, 1), coef.view(B, 1).expand(B, T), torch.zeros(B, T, dtype=torch.float64))
    assert torch.allclose(mgd.sum(1), want_mass, rtol=2 * grad_tol, atol=1e-12)
    # the rule mass of each main-chain parent equals its emission mass (the last node emits once without a rule)
    rule_mass = lg.sum(dim=(2, 3))                       # [B, L]
    emit_mass = mgd.sum(2)                               # [B, L]
    last = (ol - 1).view(B, 1)
    emit_mass = emit_mass - torch.zeros(B, L, dtype=torch.float64).scatter_(1, last, coef.view(B, 1))
    main_rows = (torch.arange(L) % 2 == 1).view(1, L)
    assert (rule_mass - emit_mass)[main_rows.expand(B, L)].abs().max() <= 2 * grad_tol * coef.abs().max()
    assert not rule_mass[~main_rows.expand(B, L)].any()
    # the oracle (float64 tables) on every sentence, end to end through the same glue, a few sentences at a time to bound
    # the host memory of the [*, L, V] float tensors
    worst = {"ll": 0.0, "match_all_grad": 0.0, "links_grad": 0.0, "logits_grad": 0.0}
    worst_bands = np.zeros((2, len(gradcheck.BANDS)))
    for s0 in range(0, B, chunk):
        sample = list(range(s0, min(B, s0 + chunk)))
        sub = {k: (v[sample] if torch.is_tensor(v) else v) for k, v in batch.items()}
        leaf = sub["logits"].float().clone().requires_grad_(True)
        lk = sub["links"].clone().requires_grad_(True)
        n_s = len(sample)
        out_mask = torch.arange(L).view(1, L) < sub["output_length"].view(n_s, 1)
        res = harness.compute_pcfg_loss(leaf * 1.0, out_mask, sub["targets"], sub["targets"].ne(synth.PAD), lk, ops=oracle_ops)
        res["match_all"].retain_grad()
        ll_o = res["ll"].detach()
        assert torch.allclose(ll[sample].cpu(), ll_o, rtol=2e-5)
        worst["ll"] = max(worst["ll"], ((ll[sample].cpu() - ll_o).abs() / ll_o.abs()).max().item())
        (res["ll"] * coef[sample].float()).sum().backward()
        lg_o, mg_o = lk.grad.double(), res["match_all"].grad.double()
        for i, b in enumerate(sample):
            err = ((lg[b] - lg_o[i]).abs().max() / lg_o[i].abs().max()).item()
            worst["links_grad"] = max(worst["links_grad"], err)
            assert err <= grad_tol, "links_grad of sentence %d: normwise error %.2e" % (b, err)
            err = ((mgd[b] - mg_o[i]).abs().max() / mg_o[i].abs().max()).item()
            worst["match_all_grad"] = max(worst["match_all_grad"], err)
            assert err <= grad_tol, "match_all_grad of sentence %d: normwise error %.2e" % (b, err)
            # every entry, relative to its own size
            worst_bands[0] = np.maximum(worst_bands[0], gradcheck.assert_elementwise(mgd[b].numpy(), mg_o[i].numpy(), "match_all_grad of sentence %d" % b))
            worst_bands[1] = np.maximum(worst_bands[1], gradcheck.assert_elementwise(lg[b].numpy(), lg_o[i].numpy(), "links_grad of sentence %d" % b))
            want_g = leaf.grad[i]
            got_g = g[b].cpu()
            # fp16 buffer: each element within fp16 rounding of the fp32 gradient (plus the rounding of the row factor)
            bound = 2 ** -9 * want_g.abs().max() + 1e-9
            err = (got_g - want_g).abs().max()
            worst["logits_grad"] = max(worst["logits_grad"], (err / want_g.abs().max()).item())
            assert err <= bound, "logits gradient of sentence %d" % b
    print("all %d sentences against the float64 oracle, worst errors: ll %.2e relative, match_all_grad %.2e, links_grad %.2e "
          "normwise, logits gradient %.2e of the row maximum (fp16 storage)"
          % (B, worst["ll"], worst["match_all_grad"], worst["links_grad"], worst["logits_grad"]))
    print("worst relative error of an entry, by its share of the sentence maximum (%s): match_all_grad %s, links_grad %s"
          % (", ".join(">= %.0e" % f for f, _ in gradcheck.BANDS), " ".join("%.1e" % e for e in worst_bands[0]),
             " ".join("%.1e" % e for e in worst_bands[1])))


def test_config2_full_size():
    _check_training_batch(synth.config2(), chunk=8)


def test_config3_full_size():
    # table entries reach ~1.8e3 here, where fp32 spacing is 1.2e-4: a plain sequential fp32 evaluation (the oracle's float
    # instantiation, which follows the reference) is 1.3e-4 .. 1.5e-4 away from float64; the kernels keep the tables
    # relative to per-column offsets and stay within the same 1e-4 as at the short lengths
    _check_training_batch(synth.config3(), chunk=4)


def test_config5_glat_alignment():
    batch = synth.config2()
    B, L, V = batch["logits"].shape
    prev = torch.full((B, L), 3, dtype=torch.int64)
    prev = prev.masked_fill(torch.arange(L).view(1, L) >= batch["output_length"].view(B, 1), synth.PAD)
    logits = batch["logits"].to(DEV)
    g1 = torch.Generator().manual_seed(7)
    got = harness.glat_alignment(logits, batch["targets"].to(DEV), prev.to(DEV), batch["links"].to(DEV), 0.5, generator=g1,
                                 noise_device="cpu")
    assert torch.equal(logits, batch["logits"].to(DEV))  # no gradient requested: logits untouched
    # oracle trace on the GPU's own inside table: bit-exact
    idx = batch["targets"].unsqueeze(1).expand(-1, L, -1)
    sel = ops._logsoftmax_gather(logits, idx.to(DEV), False)
    match = harness.eos_masked(sel, batch["output_length"].to(DEV), batch["target_length"].to(DEV))
    S_gpu, _, _, _ = ops._pcfg_loss_tables(match, batch["links"].to(DEV), batch["output_length"].to(DEV),
                                           batch["target_length"].to(DEV), 1, "test")
    m_np, l_np = match.cpu().numpy(), batch["links"].numpy()
    ol, tl = batch["output_length"].numpy(), batch["target_length"].numpy()
    _, C32 = oracle.inside_fwd(m_np, l_np, ol, tl, dtype=np.float32)
    want_tree, margin32 = oracle.best_tree(S_gpu.cpu().numpy(), C32, m_np, l_np, ol, tl, dtype=np.float32, return_margin=True)
    print("config 5, best-tree trace on the GPU's own fp32 table (entries of order 1e2): smallest arg-max margin %.3e, %d exact "
          "ties" % (margin32[:, 0].min(), margin32[:, 1].sum()))
    tree = torch.from_numpy(want_tree)
    path = tree.clone()
    path[path + 1 >= batch["targets"].shape[1] + 1] = -1
    assert torch.equal(got["path"].cpu(), path)
    # the same glue over the oracle (CPU) with the same noise: identical glancing decisions
    g2 = torch.Generator().manual_seed(7)
    oracle_ops.reset_margins()
    want = harness.glat_alignment(batch["logits"].float(), batch["targets"], prev, batch["links"], 0.5, ops=oracle_ops,
                                  generator=g2)
    print("config 5, best-tree trace of the float64 oracle: %s" % oracle_ops.margin_text("best_tree"))
    assert torch.equal(got["path"].cpu(), want["path"])
    assert torch.equal(got["keep_word_mask"].cpu(), want["keep_word_mask"])
    assert torch.equal(got["glat_prev_output_tokens"].cpu(), want["glat_prev_output_tokens"])
    assert torch.equal(got["matchmask"].cpu(), want["matchmask"])
    # the same pass as one native call, and the torch glue over the device operators, for every glance strategy of the
    # criterion: identical decisions, same random stream consumed
    for strategy, p in (("number-random", 0.5), ("number-random", 0.0), ("number-random", 1.0), ("cmlm", 0.5), (None, 0.5),
                        (None, 1.0)):
        g2 = torch.Generator().manual_seed(7)
        want = harness.glat_alignment(batch["logits"].float(), batch["targets"], prev, batch["links"], p, ops=oracle_ops,
                                      generator=g2, glance_strategy=strategy)
        if strategy is None:  # a real coin per node: some aligned nodes revealed, some not
            assert 0 < int(want["keep_word_mask"].sum()) < int((want["path"] >= 0).sum())
        for single_call in (True, False):
            g3 = torch.Generator().manual_seed(7)
            one = harness.glat_alignment(logits, batch["targets"].to(DEV), prev.to(DEV), batch["links"].to(DEV), p, generator=g3,
                                         noise_device="cpu", single_call=single_call, glance_strategy=strategy)
            assert torch.equal(logits, batch["logits"].to(DEV))
            assert torch.equal(g2.get_state(), g3.get_state())
            for key in ("path", "keep_word_mask", "glat_prev_output_tokens", "matchmask", "same_num", "glance_nums"):
                assert one[key].dtype == want[key].dtype and torch.equal(one[key].cpu(), want[key]), (strategy, p, single_call, key)
            assert torch.allclose(one["max_tree_lprob"].cpu(), want["max_tree_lprob"], rtol=2e-5)


def test_config4_viterbi_decode():
    """All 1000 sentences of the inference configuration, once as 16 length-sorted batches of 64 (the last one holds 40) and
    once one by one, through both call paths (tables + readout as separate operators, and the single native call):
    lengths and token ids bit-exact against the oracle."""
    lens = synth.config4_lengths()
    srt = torch.sort(lens)[0]
    gen = torch.Generator(device=DEV).manual_seed(3)
    masks = {}

    def case(src):
        m = 4 * src
        Lx = int(m.max())
        g = torch.Generator().manual_seed(int(src.sum()))
        links = synth.make_links(len(src), Lx, m, 1, g)
        logits = (torch.randn(len(src), Lx, 40000, device=DEV, generator=gen) * 3).half()
        ob, tok = synth.ob_and_tokens(logits)  # computed once, fed to both paths
        del logits
        if Lx not in masks:
            masks[Lx] = synth.support_masks(Lx, 1)[0]
        return ob, tok, links, m, masks[Lx]

    for what, chunks in (("16 batches of up to 64", [srt[i:i + 64] for i in range(0, len(srt), 64)]),
                         ("1000 single sentences", [lens[i:i + 1] for i in range(len(lens))])):
        oracle_ops.reset_margins()
        n_sent = 0
        for src in chunks:
            ob, tok, links, m, mask = case(src)
            want_tok, want_len = harness.viterbi_decode(ob.cpu(), tok.cpu(), links, m, mask, ops=oracle_ops)
            for single_call in (False, True):
                got_tok, got_len = harness.viterbi_decode(ob, tok, links.to(DEV), m.to(DEV), mask.to(DEV), single_call=single_call)
                assert torch.equal(got_len.cpu(), want_len)
                assert torch.equal(got_tok.cpu(), want_tok)
            n_sent += len(src)
        assert n_sent == 1000
        print("config 4, %s, Viterbi tables of the fp32 oracle (entries of order 1e2): %s" % (what, oracle_ops.margin_text("viterbi")))


def test_config2_link_scorer_full_size():
    """The link scorer at the training shape (B=40, L=128, 8 heads of 64): forward and all four gradients against the torch
    restatement evaluated in float64 on the device; prints the time of both (the restatement in fp32, as the model runs it)."""
    import time
    from oracle import extract_links_ref as ref
    B, L, H, F = 40, 128, 8, 64
    g = torch.Generator().manual_seed(0)
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 0.5).half().to(DEV) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).half().to(DEV)
    m, _ = synth._wmt_lengths(B, torch.Generator().manual_seed(1001), 10, L // 4, 32)
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= m.view(B, 1), synth.PAD).to(DEV)
    lm, rm, mc = (x.to(DEV) for x in synth.support_masks(L, 1))
    leaves = [t.double().requires_grad_(True) for t in (q, kl, kr, gate)]
    want = ref.extract_links(*leaves, prev, synth.PAD, lm, rm, mc).double()
    fin = torch.isfinite(want)
    G = torch.randn(want.shape, generator=g, dtype=torch.float64).to(DEV).masked_fill(~fin, 0)
    want.masked_fill(~fin, 0).mul(G).sum().backward()
    mine = [t.clone().requires_grad_(True) for t in (q, kl, kr, gate)]
    got = ops.pcfg_extract_links(*mine, prev, synth.PAD, lm, rm, mc)
    assert torch.equal(torch.isfinite(got), fin)
    assert torch.allclose(got.double()[fin], want.detach()[fin], rtol=2e-5, atol=2e-5)
    rows = torch.logsumexp(got.view(B, L, -1), -1)
    usable = torch.isfinite(rows)
    assert torch.allclose(rows[usable], torch.zeros_like(rows[usable]), atol=2e-5)  # every usable row is a distribution
    got.backward(G.float())
    for name, a, b in zip(("q", "kl", "kr", "gate"), mine, leaves):
        err = ((a.grad.double() - b.grad).abs().max() / b.grad.abs().max()).item()
        print("link scorer gradient %s: normwise error %.2e" % (name, err))
        assert err <= 2e-3  # gradients are returned in the inputs' fp16

    def timed(fn, reps=10):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e6

    def run(fn_links):
        ts = [t.detach().clone().requires_grad_(True) for t in (q, kl, kr, gate)]
        fn_links(*ts).backward(G.float())
    t_ours = timed(lambda: run(lambda *t: ops.pcfg_extract_links(*t, prev, synth.PAD, lm, rm, mc)))
    t_ref = timed(lambda: run(lambda *t: ref.extract_links(*t, prev, synth.PAD, lm, rm, mc).masked_fill(~fin, 0)))
    print("link scorer forward+backward: %.0f us here, %.0f us for the torch restatement" % (t_ours, t_ref))
