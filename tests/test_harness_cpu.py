"""The criterion / decoder glue (pcfg_nat_amd/harness.py) run over the CPU oracle: checks the glue itself (eos masking,
loss reduction, GLAT sampling, length selection) on the tiny plumbing configuration."""
import numpy as np
import pytest
import torch

import oracle_ops
from pcfg_nat_amd import harness, synth


def _masks(batch):
    B, L, _ = batch["logits"].shape
    out_mask = torch.arange(L).view(1, L) < batch["output_length"].view(B, 1)
    return out_mask, batch["targets"].ne(synth.PAD)


def test_eos_mask_semantics():
    match = torch.zeros(2, 6, 4)
    out = harness.eos_masked(match, torch.tensor([6, 4]), torch.tensor([4, 3]))
    assert torch.isinf(out[0, :5, 3]).all() and out[0, 5, 3] == 0
    assert torch.isinf(out[1, [0, 1, 2, 4, 5], 2]).all() and out[1, 3, 2] == 0
    assert (out[1, :, 3] == 0).all() and (out[:, :, :2] == 0).all()


def test_loss_and_gradients_config1():
    batch = synth.config1()
    out_mask, tgt_mask = _masks(batch)
    leaf = batch["logits"].clone().requires_grad_(True)
    links = batch["links"].clone().requires_grad_(True)
    res = harness.compute_pcfg_loss(leaf * 1.0, out_mask, batch["targets"], tgt_mask, links, ops=oracle_ops)
    assert torch.isfinite(res["loss"]) and int(res["invalid_nsentences"]) == 0
    res["loss"].backward()
    # d loss / d logits sums to zero over the vocabulary (softmax gradient), rows of pads get nothing
    assert leaf.grad.sum(-1).abs().max() < 1e-5
    assert torch.isfinite(links.grad).all()
    # the loss is -(ll / n).mean(): every sentence's emission posterior mass is n, so the logits gradient w.r.t. the
    # gathered columns carries total mass -1/B per sentence
    B = leaf.shape[0]
    tgt = batch["targets"]
    # finite-difference spot check through the whole glue
    eps = 1e-3
    b, p, v = 0, 5, int(tgt[0, 3])
    xp, xm = batch["logits"].clone().double(), batch["logits"].clone().double()
    xp[b, p, v] += eps
    xm[b, p, v] -= eps
    lp = harness.compute_pcfg_loss(xp, out_mask, tgt, tgt_mask, batch["links"].double(), ops=oracle_ops)["loss"]
    lm = harness.compute_pcfg_loss(xm, out_mask, tgt, tgt_mask, batch["links"].double(), ops=oracle_ops)["loss"]
    fd = float(lp - lm) / (2 * eps)
    assert abs(fd - float(leaf.grad[b, p, v])) < 1e-4 * max(1.0, abs(fd)) + 1e-6


def test_glat_alignment_is_deterministic_and_consistent():
    batch = synth.config1()
    B, L, V = batch["logits"].shape
    prev = torch.full((B, L), 3, dtype=torch.int64)  # unk everywhere, no pads: output_length = L
    outs = []
    for _ in range(2):
        gen = torch.Generator().manual_seed(7)
        outs.append(harness.glat_alignment(batch["logits"].clone(), batch["targets"], prev, batch["links"], 0.5,
                                           ops=oracle_ops, generator=gen))
    a, b = outs
    assert torch.equal(a["keep_word_mask"], b["keep_word_mask"])
    assert torch.equal(a["glat_prev_output_tokens"], b["glat_prev_output_tokens"])
    path = a["path"]
    n = batch["target_length"]
    for i in range(B):
        used = path[i][path[i] >= 0]
        assert used.tolist() == list(range(int(n[i])))
    # revealed nodes carry exactly their aligned target token, the others keep the previous token (times zero trick of
    # the reference: masked_fill(keep, 0) + oracle.masked_fill(~keep, 0))
    keep = a["keep_word_mask"]
    oracle_tok = batch["targets"].gather(-1, path.clip(min=0))
    assert torch.equal(a["glat_prev_output_tokens"][keep], oracle_tok[keep])
    assert (a["glat_prev_output_tokens"][~keep] == 3).all()
    assert (keep.sum(1) <= a["glance_nums"]).all()
    assert a["matchmask"].shape == (B, batch["targets"].shape[1], L)
    assert torch.equal(a["matchmask"].sum(-1).sum(-1), n)


def test_glance_strategies_consume_the_reference_random_stream():
    """The three glance strategies of the criterion (nat_pcfg_loss.py:231-251) over the oracle: `number-random` reveals
    round((n - same) * p) nodes chosen by a randn ranking, `cmlm` a uniform share of the target length, the default flips a
    coin per aligned node with probability (n - same) / n * p; each consumes exactly the draws the reference makes, in its
    order (randn [B,L]; rand [B] for cmlm; rand [B,L])."""
    batch = synth.config1()
    B, L, V = batch["logits"].shape
    prev = torch.full((B, L), 3, dtype=torch.int64)
    n = batch["target_length"]

    def run(strategy, p):
        gen = torch.Generator().manual_seed(11)
        out = harness.glat_alignment(batch["logits"].clone(), batch["targets"], prev, batch["links"], p, ops=oracle_ops,
                                     generator=gen, glance_strategy=strategy)
        return out, gen

    def stream_after(draws):
        gen = torch.Generator().manual_seed(11)
        for kind, shape in draws:
            (torch.randn if kind == "n" else torch.rand)(shape, generator=gen)
        return gen.get_state()

    out, gen = run("number-random", 0.5)
    assert torch.equal(gen.get_state(), stream_after([("n", (B, L)), ("u", (B, L))]))
    assert torch.equal(out["keep_word_mask"].sum(1), ((n - out["same_num"]) * 0.5 + 0.5).long())
    out, gen = run("cmlm", 0.5)
    assert torch.equal(gen.get_state(), stream_after([("n", (B, L)), ("u", (B,)), ("u", (B, L))]))
    g = torch.Generator().manual_seed(11)
    torch.randn((B, L), generator=g)
    want_nums = (n * torch.rand((B,), generator=g) + 0.5).long()
    assert torch.equal(out["glance_nums"], want_nums) and torch.equal(out["keep_word_mask"].sum(1), want_nums.clamp(max=n))
    out, gen = run(None, 1.0)
    assert torch.equal(gen.get_state(), stream_after([("u", (B, L))]))
    aligned = out["path"] >= 0
    assert not (out["keep_word_mask"] & ~aligned).any()
    u = torch.rand((B, L), generator=torch.Generator().manual_seed(11))
    share = ((n - out["same_num"]) / n * 1.0).unsqueeze(-1)
    assert torch.equal(out["keep_word_mask"], (u < share * aligned.float()))
    with pytest.raises(RuntimeError):
        run("random", 0.5)


def test_force_emit_semantics():
    """Force-emit (nat_pcfg_loss.py:116-121) over the oracle ops: revealed nodes keep only their aligned target position
    and pass no gradient; with every node marked as revealed the loss is that of the single derivation the alignment
    spells (its emissions + its links), which is computed here by hand from the path."""
    batch = synth.config1()
    out_mask, tgt_mask = _masks(batch)
    B, L, V = batch["logits"].shape
    prev = torch.full((B, L), 3, dtype=torch.int64)
    gen = torch.Generator().manual_seed(3)
    glat = harness.glat_alignment(batch["logits"].clone(), batch["targets"], prev, batch["links"], 0.5, ops=oracle_ops,
                                  generator=gen)
    mm, keep = glat["matchmask"], glat["keep_word_mask"]
    assert keep.any()
    leaf = batch["logits"].clone().requires_grad_(True)
    res = harness.compute_pcfg_loss(leaf * 1.0, out_mask, batch["targets"], tgt_mask, batch["links"], ops=oracle_ops,
                                    matchmask=mm, keep_word_mask=keep)
    res["loss"].backward()
    assert torch.isfinite(res["loss"])
    assert not leaf.grad[keep].any() and leaf.grad[~keep].any()
    off = harness.compute_pcfg_loss(batch["logits"].clone(), out_mask, batch["targets"], tgt_mask, batch["links"],
                                    ops=oracle_ops, matchmask=mm, keep_word_mask=keep, no_force_emit=True)
    plain = harness.compute_pcfg_loss(batch["logits"].clone(), out_mask, batch["targets"], tgt_mask, batch["links"],
                                      ops=oracle_ops)
    assert torch.equal(off["loss"], plain["loss"]) and float(res["loss"].detach()) > float(plain["loss"])
    # every node marked as revealed (nodes off the alignment then can emit nothing): only the aligned derivation survives
    path = glat["path"]
    all_keep = torch.ones_like(path, dtype=torch.bool)
    one = harness.compute_pcfg_loss(batch["logits"].clone(), out_mask, batch["targets"], tgt_mask, batch["links"],
                                    ops=oracle_ops, matchmask=mm, keep_word_mask=all_keep)
    logp = torch.log_softmax(batch["logits"].double(), -1)
    for b in range(B):
        nodes = [a for a in range(L) if path[b, a] >= 0]
        total = sum(float(logp[b, a, batch["targets"][b, path[b, a]]]) for a in nodes)
        mains = [a for a in nodes if a % 2 == 1]
        for a, c in zip(mains[:-1], mains[1:]):
            k = 1 if (a - 1) in nodes and a - 1 >= 1 else 0  # the leaf in front of a is on the tree: left option 1
            total += float(batch["links"][b, a, k, c])
        assert abs(float(one["ll"][b]) - total) < 1e-4 * abs(total), (b, float(one["ll"][b]), total)


def test_viterbi_decode_glue():
    batch = synth.decode_batch([6, 10, 4], seed=5, V=64, logit_dtype=torch.float32)
    ob, tok = synth.ob_and_tokens(batch["logits"])
    L = batch["links"].shape[1]
    left_mask, _, _ = synth.support_masks(L, 1)
    tokens, pred_len = harness.viterbi_decode(ob, tok, batch["links"], batch["output_length"], left_mask, ops=oracle_ops)
    assert tokens.dtype == torch.float32 and tokens.shape[0] == 3
    assert (pred_len >= 1).all() and (pred_len < batch["output_length"] // 4).all()
    # the number of emitted tokens never exceeds the predicted length (dedup and pad-skip only remove)
    assert ((tokens != synth.PAD).sum(1) <= pred_len).all()


def test_support_masks_closed_form():
    left, right, main = synth.support_masks(10, 1)
    assert main.tolist() == [False, True, False, True, False, True, False, True, False, True]
    assert left[3, 2] == 0 and left[3, 0] == 0 and left[3, 1] == 1 and left[1, 0] == 0 and left[0, 0] == 1
    assert right[1, 2:].eq(0).all() and right[2].eq(1).all()
    left3, right3, main3 = synth.support_masks(14, 3)
    assert main3.nonzero().flatten().tolist() == [1, 5, 9, 13]
    assert left3[5, 2:5].eq(0).all() and left3[3, 2] == 0 and right3[3, 4] == 0 and left3[3, 4] == 1


def test_flag_mask_cache_handles_views_and_inference_tensors():
    """Integer support masks are converted to byte flags once and found again under fresh views of the same tensor; a
    mask changed in place is converted again; tensors created under inference mode (no version counter) are converted on
    every call instead of raising."""
    from pcfg_nat_amd import custom_ops
    custom_ops._MASK_CACHE.clear()
    mask = torch.zeros(8, 8, dtype=torch.int64)
    mask[2, 3] = 1
    a = custom_ops._as_flag_mask(mask[:6, :6])
    b = custom_ops._as_flag_mask(mask[:6, :6])  # a fresh view object of the same storage
    assert a is b and a.dtype == torch.bool and bool(a[2, 3]) and int(a.sum()) == 1
    assert len(custom_ops._MASK_CACHE) == 1
    mask[4, 4] = 1  # in place: the version counter moves on
    c = custom_ops._as_flag_mask(mask[:6, :6])
    assert c is not a and int(c.sum()) == 2
    with torch.inference_mode():
        inf = torch.ones(4, 4, dtype=torch.int64)
    d = custom_ops._as_flag_mask(inf)
    assert d.dtype == torch.bool and bool(d.all())
    flags = torch.ones(4, 4, dtype=torch.bool)
    assert custom_ops._as_flag_mask(flags) is flags or torch.equal(custom_ops._as_flag_mask(flags), flags)
