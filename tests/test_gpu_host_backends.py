"""The host side of the training operators (and of the link scorer with its products inside the kernels) exists twice - as C++ autograd nodes in the torch extension (what runs by
default) and as the Python Functions of ``custom_ops`` over ctypes.  Both enqueue the same kernels with the same arguments,
so every result must be bit-identical; the contract checks (in-place buffer, single backward, loud errors) hold in both."""
import pytest
import torch

from pcfg_nat_amd import _lib, custom_ops as ops, harness, synth

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(params=["extension", "python"])
def backend(request):
    before = ops.host_backend()
    ops.host_backend(request.param)
    yield request.param
    ops.host_backend(before)


def _batch():
    batch = synth.training_batch(5, 64, 12, 700, [64, 40, 22, 8, 64], [12, 9, 12, 12, 2], seed=43, logit_scale=2.0,
                                 logit_dtype=torch.float16)
    B, L, _ = batch["logits"].shape
    out_mask = (torch.arange(L).view(1, L) < batch["output_length"].view(B, 1)).to(DEV)
    return batch, out_mask


def _run_operator_path(batch, out_mask, scale):
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    links = batch["links"].to(DEV).requires_grad_(True)
    tgt = batch["targets"].to(DEV)
    res = harness.compute_pcfg_loss(leaf.half(), out_mask, tgt, tgt.ne(synth.PAD), links)
    (res["loss"] * scale).backward()
    return res["loss"].detach(), res["ll"].detach(), leaf.grad, links.grad


def _run_criterion(batch, scale, masks=None):
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    links = batch["links"].to(DEV).requires_grad_(True)
    ol, tl = batch["output_length"].to(DEV), batch["target_length"].to(DEV)
    mm, keep = masks if masks is not None else (None, None)
    loss, ll, invalid = ops.pcfg_criterion(leaf.half(), batch["targets"].to(DEV), links, ol, tl, mm, keep)
    (loss * scale).backward()
    return loss.detach(), ll.detach(), invalid.detach(), leaf.grad, links.grad


def test_extension_is_the_default_and_loads():
    assert ops.host_backend() == "extension"
    ext = _lib.load_ext()
    assert ext.abi_version() == _lib.load().pcfgnat_abi_version()


def test_backends_give_identical_results():
    batch, out_mask = _batch()
    results = {}
    before = ops.host_backend()
    try:
        for name in ("extension", "python"):
            ops.host_backend(name)
            results[name] = (_run_operator_path(batch, out_mask, 128.0), _run_criterion(batch, 128.0))
    finally:
        ops.host_backend(before)
    for a, b in zip(results["extension"], results["python"]):
        for x, y in zip(a, b):
            assert torch.equal(x, y)
    # and the two paths agree with each other to rounding (one fp16 rounding step on the logits' gradient)
    op, cr = results["extension"]
    assert torch.allclose(cr[0], op[0], rtol=1e-6) and torch.allclose(cr[1], op[1], rtol=1e-6)
    assert torch.allclose(cr[4], op[3], rtol=1e-5, atol=1e-7)
    assert torch.allclose(cr[3], op[2], rtol=2 ** -9, atol=2 ** -24)


def test_criterion_force_emit_and_no_grad(backend):
    batch, out_mask = _batch()
    B, L, _ = batch["logits"].shape
    tgt = batch["targets"].to(DEV)
    prev = torch.full((B, L), 3, dtype=torch.int64, device=DEV).masked_fill(~out_mask, synth.PAD)
    glat = harness.glat_alignment(batch["logits"].to(DEV).clone(), tgt, prev, batch["links"].to(DEV), 0.5,
                                  generator=torch.Generator().manual_seed(5), noise_device="cpu")
    loss, ll, invalid, g_logits, g_links = _run_criterion(batch, 1.0, (glat["matchmask"], glat["keep_word_mask"]))
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    links = batch["links"].to(DEV).requires_grad_(True)
    res = harness.compute_pcfg_loss(leaf.half(), out_mask, tgt, tgt.ne(synth.PAD), links, matchmask=glat["matchmask"],
                                    keep_word_mask=glat["keep_word_mask"])
    res["loss"].backward()
    assert torch.allclose(loss, res["loss"].detach(), rtol=1e-6)
    assert torch.allclose(g_links, links.grad, rtol=1e-5, atol=1e-9)
    assert torch.allclose(g_logits, leaf.grad, rtol=2 ** -9, atol=2 ** -22)
    # nothing requires a gradient: same loss, no graph
    with torch.no_grad():
        loss2, ll2, _ = ops.pcfg_criterion(batch["logits"].to(DEV).clone(), tgt, batch["links"].to(DEV),
                                           batch["output_length"].to(DEV), batch["target_length"].to(DEV))
    assert not loss2.requires_grad
    plain = harness.compute_pcfg_loss(batch["logits"].to(DEV).clone(), out_mask, tgt, tgt.ne(synth.PAD), batch["links"].to(DEV))
    assert torch.allclose(loss2, plain["loss"], rtol=1e-6) and torch.allclose(ll2, plain["ll"], rtol=1e-6)


def test_contract_of_the_in_place_operators(backend):
    batch, _ = _batch()
    B, L, V = batch["logits"].shape
    tgt = batch["targets"].to(DEV)
    idx = tgt.unsqueeze(1).expand(-1, L, -1)
    leaf = batch["logits"].to(DEV).float().requires_grad_(True)
    x = leaf * 1.0
    out, sel = ops.dag_logsoftmax_gather_inplace(x, idx)
    assert out.data_ptr() == x.data_ptr() and sel.dtype == torch.float32 and sel.requires_grad
    sel.sum().backward(retain_graph=True)
    with pytest.raises((RuntimeError, AssertionError), match="twice"):
        sel.sum().backward()
    # the buffer handed back must not be used again
    leaf2 = batch["logits"].to(DEV).float().requires_grad_(True)
    out, sel = ops.dag_logsoftmax_gather_inplace(leaf2 * 1.0, idx)
    with pytest.raises((RuntimeError, AssertionError), match="reuse"):
        (sel.sum() + out.sum()).backward()
    # no gradient requested: buffer untouched, no graph
    y = batch["logits"].to(DEV).float()
    keep = y.clone()
    out, sel = ops.dag_logsoftmax_gather_inplace(y, idx)
    assert torch.equal(y, keep) and not sel.requires_grad
    with pytest.raises(RuntimeError, match="select_idx should be long"):
        ops.dag_logsoftmax_gather_inplace(y, idx.int())
    with pytest.raises(RuntimeError, match="not contiguous"):
        ops.dag_logsoftmax_gather_inplace(y.transpose(0, 1), idx.transpose(0, 1))
    with pytest.raises(RuntimeError, match="links"):
        ops.cuda_pcfg_loss(sel.detach(), batch["links"].to(DEV)[:, :, :, :-1], batch["output_length"].to(DEV),
                           batch["target_length"].to(DEV))
    with pytest.raises(RuntimeError, match="lengths should be long"):
        ops.cuda_pcfg_loss(sel.detach(), batch["links"].to(DEV), batch["output_length"].to(DEV).int(),
                           batch["target_length"].to(DEV))
    ops.CUDAPCFGLossFunc.config = 5
    try:
        with pytest.raises(RuntimeError, match="config should be 1~4"):
            ops.cuda_pcfg_loss(sel.detach(), batch["links"].to(DEV), batch["output_length"].to(DEV), batch["target_length"].to(DEV))
    finally:
        ops.CUDAPCFGLossFunc.config = 1
    # the loss op: gradient only when asked for, the eager backward's gradients scaled by the upstream one
    match = harness.eos_masked(sel.detach(), batch["output_length"].to(DEV), batch["target_length"].to(DEV)).requires_grad_(True)
    ll = ops.cuda_pcfg_loss(match, batch["links"].to(DEV), batch["output_length"].to(DEV), batch["target_length"].to(DEV))
    w = torch.linspace(0.5, 1.5, B, device=DEV)
    ll.backward(w)
    ll1 = ops.cuda_pcfg_loss(match.detach().requires_grad_(True), batch["links"].to(DEV), batch["output_length"].to(DEV),
                             batch["target_length"].to(DEV))
    assert torch.equal(ll1, ll.detach())
    assert match.grad is not None and torch.isfinite(match.grad).all()


def test_link_scorer_backends_give_identical_results():
    """pcfg_extract_links through the C++ node and through the Python Function: same kernels, same arguments."""
    B, L, H, F = 3, 64, 4, 32
    g = torch.Generator().manual_seed(5)
    chunks = [(torch.randn(B, L, H, F, generator=g) * 0.5).half().to(DEV) for _ in range(3)]
    gate = torch.randn(B, L, H, generator=g).half().to(DEV)
    m = torch.tensor([64, 40, 24])
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= m.view(B, 1), synth.PAD).to(DEV)
    lm, rm, mc = (x.to(DEV) for x in synth.support_masks(L, 1))
    G = torch.randn(B, L, 2, L, generator=g).to(DEV)
    results = {}
    before = ops.host_backend()
    try:
        for name in ("extension", "python"):
            ops.host_backend(name)
            ts = [t.detach().requires_grad_(True) for t in chunks + [gate]]
            links = ops.pcfg_extract_links(*ts, prev, synth.PAD, lm, rm, mc)
            links.backward(G.masked_fill(~torch.isfinite(links.detach()), 0))
            results[name] = [links.detach()] + [t.grad for t in ts]
            with torch.no_grad():  # (no backward to prepare: the masks per parent are not written)
                assert torch.equal(ops.pcfg_extract_links(*chunks, gate, prev, synth.PAD, lm, rm, mc), links.detach())
    finally:
        ops.host_backend(before)
    for a, b in zip(results["extension"], results["python"]):
        assert a.dtype == b.dtype and torch.equal(a, b)


def test_decode_backends_give_identical_results(backend):
    """The single-call Viterbi decode through the C++ enqueue function and through the Python wrapper over ctypes: the
    oracle's tokens and lengths from both, from the logits (with the front-end's node scores and tokens) and from the node
    scores; a batch, one sentence, an empty batch; the same loud errors."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    import oracle_ops
    from pcfg_nat_amd import harness
    batch = synth.decode_batch([30, 8, 51, 3], seed=11, V=300)
    L = batch["links"].shape[1]
    lm = synth.support_masks(L, 1)[0]
    ob, tok = synth.ob_and_tokens(batch["logits"])
    want_tok, want_len = harness.viterbi_decode(ob, tok, batch["links"], batch["output_length"], lm, ops=oracle_ops, beta=0.8)
    logits, links, ol, lmd = batch["logits"].to(DEV), batch["links"].to(DEV), batch["output_length"].to(DEV), lm.to(DEV)
    got_tok, got_len, scores, toks = ops.pcfg_viterbi_decode_logits(logits, links, ol, lmd, synth.PAD, 0.8, return_nodes=True)
    assert got_tok.dtype == torch.float32 and torch.equal(got_tok.cpu(), want_tok) and torch.equal(got_len.cpu(), want_len)
    assert torch.equal(toks.cpu(), tok) and torch.allclose(scores.cpu(), ob, atol=2e-6)
    got_tok, got_len = ops.pcfg_viterbi_decode(scores, links, ol, toks.int(), lmd.bool(), synth.PAD, 0.8)  # (dtypes are converted)
    assert torch.equal(got_tok.cpu(), want_tok) and torch.equal(got_len.cpu(), want_len)
    # one sentence: the row comes back as a view, still the oracle's tokens
    one = synth.decode_batch([19], seed=12, V=300)
    L1 = one["links"].shape[1]
    lm1 = synth.support_masks(L1, 1)[0]
    ob1, tok1 = synth.ob_and_tokens(one["logits"])
    w_tok, w_len = harness.viterbi_decode(ob1, tok1, one["links"], one["output_length"], lm1, ops=oracle_ops)
    g_tok, g_len = ops.pcfg_viterbi_decode_logits(one["logits"].to(DEV), one["links"].to(DEV), one["output_length"].to(DEV), lm1.to(DEV),
                                                  synth.PAD)
    assert g_tok.is_contiguous() and torch.equal(g_tok.cpu(), w_tok) and torch.equal(g_len.cpu(), w_len)
    # nothing to decode
    e_tok, e_len = ops.pcfg_viterbi_decode_logits(logits[:0], links[:0], ol[:0], lmd, synth.PAD)
    assert e_tok.shape == (0, 0) and e_len.shape == (0,)
    with pytest.raises(RuntimeError, match="float16 or float32"):
        ops.pcfg_viterbi_decode_logits(logits.double(), links, ol, lmd, synth.PAD)
    with pytest.raises(RuntimeError, match="lengths should be long"):
        ops.pcfg_viterbi_decode_logits(logits, links, ol.int(), lmd, synth.PAD)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.pcfg_viterbi_decode_logits(logits, links.cpu(), ol, lmd, synth.PAD)
    with pytest.raises(RuntimeError, match="does not match"):
        ops.pcfg_viterbi_decode_logits(logits, links[:, :-2], ol, lmd, synth.PAD)
