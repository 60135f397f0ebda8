"""Pins for the CPU oracle's inside forward / backward (oracle/pcfg_oracle_body.h).

The reference (fs_plugins/custom_ops) holds no tests or golden vectors for this path, so the oracle is pinned by what
the mathematics fixes: brute-force enumeration of derivations on tiny graphs, the textbook DAG forward algorithm for
the special case without left children, central finite differences, and the mass-conservation invariants.
"""
import math

import numpy as np
import pytest
import torch

import bruteforce as bf
from oracle import oracle
from pcfg_nat_amd import synth

NINF = -math.inf


def random_links(rng, L, m, ml, p_drop=0.2, generic_local=False):
    """Links with the grammar's structural support (not normalised): finite for main parents a<c (c main), optionally
    also for local parents with a right child in their own group; random entries dropped to -inf."""
    links = np.full((L, ml + 1, L), NINF)
    for a in range(1, m):
        if bf.is_main(a, ml):
            for c in range(a + ml + 1, m, ml + 1):
                for k in range(ml + 1):
                    if k and a - k < 1:
                        continue
                    if rng.random() > p_drop:
                        links[a, k, c] = rng.normal() - 1.0
        elif generic_local:
            lo = bf.group_lo(a, ml)
            for c in range(a + 1, min(lo + ml + 1, m)):
                for k in range(ml + 1):
                    if k and (a - k < 1 or bf.is_main(a - k, ml)):
                        continue
                    if rng.random() > p_drop:
                        links[a, k, c] = rng.normal() - 1.0
    return links


def oracle_ll(match, links, m, n, dtype=np.float64):
    S, C = oracle.inside_fwd(match[None], links[None], np.array([m]), np.array([n]), dtype=dtype)
    return S[0, 0, 0], S, C


@pytest.mark.parametrize("ml,L,n_list", [(1, 12, [2, 3, 5, 7, 9]), (3, 14, [2, 4, 5, 7]), (3, 18, [6, 8])])
def test_loglik_matches_enumeration(ml, L, n_list):
    rng = np.random.default_rng(10 * ml + L)
    for n in n_list:
        for m in {L, L - (ml + 1)}:
            T = n + 1
            match = rng.normal(size=(L, T)) - 2.0
            links = random_links(rng, L, m, ml, generic_local=(ml > 1))
            want = bf.inside_loglik(match.tolist(), links.tolist(), m, n, ml)
            got, _, _ = oracle_ll(match, links, m, n)
            if want == NINF:
                assert got == NINF
            else:
                assert abs(got - want) < 1e-10, (ml, L, m, n, got, want)


def test_local_composites_are_exercised():
    """The ml=3 generic-support case must actually use gap>=2 local derivations, otherwise the pin above is vacuous."""
    rng = np.random.default_rng(5)
    ml, L, m, n = 3, 14, 14, 6
    links = random_links(rng, L, m, ml, p_drop=0.0, generic_local=True)
    ders = bf.main_derivations(1, m, ml, links.tolist(), n)
    assert any(any(not bf.is_main(x, ml) and not bf.is_main(y, ml) and y == x + 1 for x, y in zip(d[0], d[0][1:]))
               for d in ders if len(d[0]) == n)
    match = rng.normal(size=(L, n)) - 2.0
    masked = links.copy()
    for a in range(L):
        if not bf.is_main(a, ml):
            masked[a] = NINF
    a1, _, _ = oracle_ll(match, links, m, n)
    a2, _, _ = oracle_ll(match, masked, m, n)
    assert a1 > a2 + 1e-6


@pytest.mark.parametrize("ml", [1, 3])
def test_dag_special_case(ml):
    """Without left children the grammar is the DA-Transformer DAG; compare with a left-to-right forward pass."""
    rng = np.random.default_rng(3)
    g = ml + 1
    L = 2 + g * 12
    for m, n in [(L, 9), (L - g, 10), (2 + g * 3, 4)]:
        match = rng.normal(size=(L, n)) - 3.0
        links = random_links(rng, L, m, ml, p_drop=0.03 if m > 8 * g else 0.0)
        links[:, 1:, :] = NINF
        want = bf.dag_forward(match.tolist(), links.tolist(), m, n, ml)
        got, _, _ = oracle_ll(match, links, m, n)
        assert math.isfinite(want) and abs(got - want) < 1e-10


def test_impossible_target_is_minus_inf_with_zero_grads():
    b = synth.training_batch(2, 12, 9, 50, [12, 8], [9, 9], seed=4)
    sel = torch.log_softmax(b["logits"].double(), -1).gather(-1, b["targets"].unsqueeze(1).expand(-1, 12, -1)).numpy()
    S, C = oracle.inside_fwd(sel, b["links"].numpy(), b["output_length"].numpy(), b["target_length"].numpy())
    # sentence 1 has 4 main-chain nodes and 3 leaves usable -> at most 7 tokens < 9
    assert np.isfinite(S[0, 0, 0]) and S[1, 0, 0] == NINF
    mg, lg = oracle.inside_bwd(np.ones(2), S, C, sel, b["links"].numpy(), b["output_length"].numpy(),
                               b["target_length"].numpy())
    assert np.all(mg[1] == 0) and np.all(lg[1] == 0)
    assert np.isfinite(mg).all() and np.isfinite(lg).all()


def _fd_check(match, links, m, n, ml, rng, n_probe=40, eps=1e-6):
    ll, S, C = oracle_ll(match, links, m, n)
    assert np.isfinite(ll)
    mg, lg = oracle.inside_bwd(np.ones(1), S, C, match[None], links[None], np.array([m]), np.array([n]))
    mg, lg = mg[0], lg[0]
    fin_m = np.argwhere(np.isfinite(match))
    fin_l = np.argwhere(np.isfinite(links))
    worst = 0.0
    for _ in range(n_probe):
        a, i = fin_m[rng.integers(len(fin_m))]
        mp, mm = match.copy(), match.copy()
        mp[a, i] += eps
        mm[a, i] -= eps
        fd = (oracle_ll(mp, links, m, n)[0] - oracle_ll(mm, links, m, n)[0]) / (2 * eps)
        worst = max(worst, abs(fd - mg[a, i]))
        a, k, c = fin_l[rng.integers(len(fin_l))]
        lp, lm = links.copy(), links.copy()
        lp[a, k, c] += eps
        lm[a, k, c] -= eps
        fd = (oracle_ll(match, lp, m, n)[0] - oracle_ll(match, lm, m, n)[0]) / (2 * eps)
        worst = max(worst, abs(fd - lg[a, k, c]))
    return worst, mg, lg


@pytest.mark.parametrize("ml,L,m,n,generic", [(1, 14, 14, 8, False), (1, 14, 10, 5, False), (3, 18, 18, 7, True),
                                                (3, 18, 14, 5, False)])
def test_gradient_finite_differences(ml, L, m, n, generic):
    rng = np.random.default_rng(100 + ml + m)
    match = rng.normal(size=(L, n + 1)) - 2.0
    match[:, n - 1] = NINF  # eos column: only the last node may emit it (nat_pcfg_loss.py:111-115)
    match[m - 1, n - 1] = -0.3
    links = random_links(rng, L, m, ml, p_drop=0.15, generic_local=generic)
    worst, mg, lg = _fd_check(match, links, m, n, ml, rng)
    assert worst < 2e-7, worst


@pytest.mark.parametrize("ml", [1, 3])
def test_gradient_invariants(ml):
    """Each target token is emitted by exactly one node => sum_a match_grad[a,t] = grad_output for t<n; every non-final
    emission by a main-chain node is accompanied by exactly one rule => sum_{k,c} links_grad[a] = sum_t match_grad[a]
    (minus the final emission for the last node)."""
    g = ml + 1
    L = 2 + g * 10
    B, T, V = 3, 9, 40
    m = [L, L - g, L - 2 * g]
    n = [9, 7, 8]
    b = synth.training_batch(B, L, T, V, m, n, seed=11, ml=ml)
    sel = torch.log_softmax(b["logits"].double(), -1).gather(-1, b["targets"].unsqueeze(1).expand(-1, L, -1)).numpy()
    links = b["links"].double().numpy()
    ol, tl = b["output_length"].numpy(), b["target_length"].numpy()
    S, C = oracle.inside_fwd(sel, links, ol, tl)
    assert np.isfinite(S[:, 0, 0]).all()
    gout = np.array([1.0, 0.5, -2.0])
    mg, lg = oracle.inside_bwd(gout, S, C, sel, links, ol, tl)
    for bi in range(B):
        col = mg[bi].sum(0)
        assert np.allclose(col[:n[bi]], gout[bi], rtol=1e-10)
        assert np.all(col[n[bi]:] == 0)
        for a in range(1, m[bi], g):
            rule_mass = lg[bi, a].sum()
            emit_mass = mg[bi, a].sum()
            if a == m[bi] - 1:
                assert abs(rule_mass) < 1e-12 and abs(emit_mass - gout[bi]) < 1e-10
            else:
                assert abs(rule_mass - emit_mass) < 1e-10
        # pads and node 0 receive nothing
        assert np.all(mg[bi, m[bi]:] == 0) and np.all(mg[bi, 0] == 0)


def test_f32_instantiation_tracks_f64():
    b = synth.config1()
    L = 32
    sel = torch.log_softmax(b["logits"].double(), -1).gather(-1, b["targets"].unsqueeze(1).expand(-1, L, -1)).numpy()
    links = b["links"].numpy()
    ol, tl = b["output_length"].numpy(), b["target_length"].numpy()
    S64, C64 = oracle.inside_fwd(sel, links, ol, tl, dtype=np.float64)
    S32, C32 = oracle.inside_fwd(sel, links, ol, tl, dtype=np.float32)
    assert np.allclose(S32[:, 0, 0], S64[:, 0, 0], rtol=1e-5)
    mg64, lg64 = oracle.inside_bwd(np.ones(2), S64, C64, sel, links, ol, tl, dtype=np.float64)
    mg32, lg32 = oracle.inside_bwd(np.ones(2), S32, C32, sel, links, ol, tl, dtype=np.float32)
    assert np.allclose(mg32, mg64, rtol=1e-3, atol=1e-5) and np.allclose(lg32, lg64, rtol=1e-3, atol=1e-5)
