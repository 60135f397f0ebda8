"""Brute-force enumerators used to pin the CPU oracle.  Nothing here shares code or index arithmetic with the oracle:
derivations are enumerated as explicit objects from the grammar's meaning and scored by multiplying rule and emission
probabilities.

Grammar (reference: fs_plugins/custom_ops/pcfg_loss.cu:84-224, 262-349):
  * a main-chain node ``a`` (ids 1, ml+2, 2ml+3, ...) rewrites as (left, a, right): ``left`` is empty ("null", rule index
    k=0) or a local node ``a-k`` (k=1..ml, ``a-k >= 1``); ``right`` is a main-chain node ``c >= a`` (``c < m``);
    the last node ``m-1`` may instead just emit the final token.
  * a local node is a leaf when its offset inside its group is odd, or rewrites as (left, itself, right) with ``right`` a
    local node of the same group further right and ``left`` empty or a node at distance <= ml to its left.
  * the yield, in order, is left-yield, the node itself, right-yield; token ``i`` of the target is emitted by the i-th
    node of the yield with log-prob ``match[node][i]``; rule (a,k,c) costs ``links[a][k][c]``.
"""
import itertools
import math


def is_main(a, ml):
    return a >= 1 and (a - 1) % (ml + 1) == 0


def group_lo(a, ml):
    return ((a - 1) // (ml + 1)) * (ml + 1) + 1


def local_derivations(b, m, ml, links, max_tokens):
    """All derivations rooted at local node ``b``: list of (yield tuple, rule log-prob)."""
    out = []
    lo = group_lo(b, ml)
    hi = lo + ml + 1
    if (b - lo) % 2 == 1:
        out.append(((b,), 0.0))
    if max_tokens < 2:
        return out
    for c in range(b + 1, min(hi, m)):
        for rd_yield, rd_lp in local_derivations(c, m, ml, links, max_tokens - 1):
            for k in range(0, ml + 1):
                if k == 0:
                    lefts = [((), 0.0)]
                else:
                    bl = b - k
                    if bl < 1 or is_main(bl, ml):
                        continue
                    lefts = local_derivations(bl, m, ml, links, max_tokens - 1 - len(rd_yield))
                w = links[b][k][c]
                if w == -math.inf:
                    continue
                for ld_yield, ld_lp in lefts:
                    y = ld_yield + (b,) + rd_yield
                    if len(y) <= max_tokens:
                        out.append((y, ld_lp + rd_lp + w))
    return out


def main_derivations(a, m, ml, links, max_tokens, allow_composite_local=True):
    """All derivations rooted at main-chain node ``a`` that end with the last node ``m-1`` emitting alone:
    list of (yield tuple, rule log-prob, rules tuple)."""
    out = []
    if a == m - 1:
        out.append(((a,), 0.0, ()))
    if max_tokens < 2:
        return out
    c = a
    while c < m:
        if c >= a:
            for k in range(0, ml + 1):
                if k == 0:
                    lefts = [((), 0.0)]
                else:
                    bl = a - k
                    if bl < 1:
                        continue
                    lefts = local_derivations(bl, m, ml, links, ml if allow_composite_local else 1)
                    # a local left child may derive at most ml tokens (the tables hold gaps 0..ml for main parents)
                    lefts = [(y, lp) for (y, lp) in lefts if len(y) <= ml]
                w = links[a][k][c]
                if w != -math.inf:
                    for ly, llp in lefts:
                        budget = max_tokens - len(ly) - 1
                        if budget < 1:
                            continue
                        if c == a:
                            # self child: only sensible with a finite self link, which callers never set; skip to
                            # avoid infinite recursion.
                            continue
                        for ry, rlp, rr in main_derivations(c, m, ml, links, budget, allow_composite_local):
                            out.append((ly + (a,) + ry, llp + w + rlp, ((a, k, c),) + rr))
        c += ml + 1
    return out


def inside_loglik(match, links, m, n, ml):
    """log sum over all derivations from the root (node 1) that yield exactly n tokens."""
    total = []
    for y, lp, _ in main_derivations(1, m, ml, links, n):
        if len(y) != n:
            continue
        # local composite spans must end before the last token and obey the table bound i < n-gap-1; with the yields
        # built above that is automatic except for the bound, which we re-check from meaning: a local subtree of g>=2
        # tokens starting at token i needs i + g < n - 1.
        e = sum(match[node][i] for i, node in enumerate(y))
        total.append(lp + e)
    total = [t for t in total if t != -math.inf and not math.isnan(t)]
    if not total:
        return -math.inf
    mx = max(total)
    return mx + math.log(sum(math.exp(t - mx) for t in total))


def viterbi_best(ob, links, m, ml, max_len):
    """For every length: (best score, yield) over derivations from the root with only leaf local children
    (with the model's masks local composites are impossible)."""
    best = {}
    for y, lp, _ in main_derivations(1, m, ml, links, max_len, allow_composite_local=False):
        sc = lp + sum(ob[node] for node in y)
        if sc == -math.inf or math.isnan(sc):
            continue
        ln = len(y)
        if ln not in best or sc > best[ln][0]:
            best[ln] = (sc, y)
    return best


def lse(vals):
    vals = [v for v in vals if v != -math.inf]
    if not vals:
        return -math.inf
    mx = max(vals)
    return mx + math.log(sum(math.exp(v - mx) for v in vals))


def dag_forward(match, links, m, n, ml):
    """Textbook left-to-right forward algorithm of a DAG with emissions (the special case of the grammar in which no
    left child is ever taken): alpha[i][a] = match[a][i] + LSE_{p<a}(alpha[i-1][p] + links[p][0][a]) over main-chain
    nodes; the answer is alpha[n-1][m-1].  It runs in the opposite direction to the suffix tables of the kernels."""
    mains = [a for a in range(1, m) if is_main(a, ml)]
    alpha = {a: -math.inf for a in mains}
    alpha[1] = match[1][0]
    for i in range(1, n):
        new = {}
        for a in mains:
            new[a] = match[a][i] + lse([alpha[p] + links[p][0][a] for p in mains if p < a])
        alpha = new
    return alpha[m - 1]
