"""Pin for the oracle's logsoftmax_gather: the library routine torch.log_softmax(...).gather(...) in float64, the
softmax write-back against torch.softmax, and the stride-0 expanded index view the criterion passes
(fs_plugins/criterions/nat_pcfg_loss.py:109)."""
import numpy as np
import torch

from oracle import oracle


def test_lsg_matches_torch_with_expanded_indices():
    g = torch.Generator().manual_seed(0)
    B, L, V, T = 3, 5, 97, 7
    x = torch.randn(B, L, V, generator=g, dtype=torch.float64) * 3
    tgt = torch.randint(0, V, (B, T), generator=g)
    idx = tgt.unsqueeze(1).expand(-1, L, -1)
    assert idx.stride(1) == 0
    sel, probs = oracle.lsg_fwd(x.numpy(), idx.numpy(), want_probs=True)
    want = torch.log_softmax(x, -1).gather(-1, idx)
    assert np.allclose(sel, want.numpy(), rtol=1e-12, atol=1e-12)
    assert np.allclose(probs, torch.softmax(x, -1).numpy(), rtol=1e-12, atol=1e-15)
    # a genuinely 3-d, non-contiguous index tensor
    idx2 = torch.randint(0, V, (B, T, L), generator=g).transpose(1, 2)
    sel2, _ = oracle.lsg_fwd(x.numpy(), idx2.numpy())
    assert np.allclose(sel2, torch.log_softmax(x, -1).gather(-1, idx2).numpy(), rtol=1e-12, atol=1e-12)


def test_lsg_f32_and_half_inputs():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(2, 4, 512, generator=g) * 2).half()
    idx = torch.randint(0, 512, (2, 4, 6), generator=g)
    sel, _ = oracle.lsg_fwd(x.numpy(), idx.numpy(), dtype=np.float32)
    want = torch.log_softmax(x.float(), -1).gather(-1, idx)
    assert np.allclose(sel, want.numpy(), rtol=1e-5, atol=1e-5)


def test_lsg_bwd_is_the_gradient():
    """Autograd of the library expression pins the backward restatement."""
    g = torch.Generator().manual_seed(4)
    B, L, V, T = 2, 3, 50, 6
    x = torch.randn(B, L, V, generator=g, dtype=torch.float64, requires_grad=True)
    tgt = torch.randint(0, V, (B, T), generator=g)
    tgt[:, 4] = tgt[:, 2]
    idx = tgt.unsqueeze(1).expand(-1, L, -1)
    w = torch.randn(B, L, T, generator=g, dtype=torch.float64)
    (torch.log_softmax(x, -1).gather(-1, idx) * w).sum().backward()
    _, probs = oracle.lsg_fwd(x.detach().numpy(), idx.numpy(), want_probs=True)
    got = oracle.lsg_bwd(probs, idx.numpy(), w.numpy())
    assert np.allclose(got, x.grad.numpy(), rtol=1e-12, atol=1e-14)
