"""Pins for the torch restatement of the link scorer (oracle/extract_links_ref.py): explicit float64 loops with their own
index arithmetic, normalisation of every usable row, and the support of the result."""
import math

import pytest
import torch

from oracle import extract_links_ref as ref
from pcfg_nat_amd import synth


def _case(B, L, H, F, ms, seed):
    g = torch.Generator().manual_seed(seed)
    q, kl, kr = (torch.randn(B, L, H, F, generator=g) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g)
    m = torch.tensor(ms)
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= m.view(B, 1), synth.PAD)
    lm, rm, mc = synth.support_masks(L, 1)
    return q, kl, kr, gate, prev, lm, rm, mc, m


@pytest.mark.parametrize("L,ms", [(10, [10, 6]), (14, [14, 8, 4])])
def test_tensor_expression_matches_explicit_loops(L, ms):
    q, kl, kr, gate, prev, lm, rm, mc, m = _case(len(ms), L, 3, 4, ms, seed=L)
    got = ref.extract_links(q, kl, kr, gate, prev, synth.PAD, lm, rm, mc).double()
    want = ref.extract_links_loops(q, kl, kr, gate, prev, synth.PAD, lm, rm, mc)
    assert torch.equal(torch.isfinite(got), torch.isfinite(want))
    fin = torch.isfinite(want)
    assert fin.any()
    assert torch.allclose(got[fin], want[fin], rtol=1e-5, atol=1e-5)


def test_rows_are_normalised_and_supported_like_the_synthetic_links():
    L, ms = 18, [18, 12]
    q, kl, kr, gate, prev, lm, rm, mc, m = _case(2, L, 4, 8, ms, seed=1)
    links = ref.extract_links(q, kl, kr, gate, prev, synth.PAD, lm, rm, mc)
    mass = torch.logsumexp(links.view(2, L, -1), -1)
    usable = torch.isfinite(mass)
    assert torch.allclose(mass[usable], torch.zeros_like(mass[usable]), atol=1e-5)
    # same support as the synthetic generator of the benchmark inputs: odd parents a < m-1, odd children a < c < m
    want = torch.isfinite(synth.make_links(2, L, m, 1, torch.Generator().manual_seed(0)))
    assert torch.equal(torch.isfinite(links), want)
