"""Independent ground truth for the lattice recursion, used to pin the oracle.

Nothing here shares code with ``oracle/``: path enumeration, a float64 numpy
dynamic programme written from the recurrence, a differentiable torch
``logaddexp`` programme, and binomial closed forms.
"""
import itertools
import math

import numpy as np
import torch


def enumerate_paths(px, py, s0, t0, s1, t1, modified):
    """log-sum over every monotone path from (s0,t0) to (s1,t1), float64.

    px: [S][T1], py: [S+1][T] nested sequences / arrays for ONE utterance.
    A regular x-step (s,t)->(s+1,t) costs px[s][t]; a modified x-step
    (s,t)->(s+1,t+1) costs px[s][t]; a y-step (s,t)->(s,t+1) costs py[s][t].
    """
    ns, nt = s1 - s0, t1 - t0
    total = -math.inf
    if modified:
        # choose which of the nt frame advances also consume a symbol
        if ns > nt:
            return -math.inf
        for xs in itertools.combinations(range(nt), ns):
            xs = set(xs)
            s, t, acc = s0, t0, 0.0
            for k in range(nt):
                if k in xs:
                    acc += float(px[s][t])
                    s += 1
                else:
                    acc += float(py[s][t])
                t += 1
            total = np.logaddexp(total, acc)
        return float(total)
    for xs in itertools.combinations(range(ns + nt), ns):
        xs = set(xs)
        s, t, acc = s0, t0, 0.0
        for k in range(ns + nt):
            if k in xs:
                acc += float(px[s][t])
                s += 1
            else:
                acc += float(py[s][t])
                t += 1
        total = np.logaddexp(total, acc)
    return float(total)


def dp_numpy(px, py, s0, t0, s1, t1, modified):
    """float64 table p[s][t] over the window (nan elsewhere) for one utterance."""
    px = np.asarray(px, dtype=np.float64)
    py = np.asarray(py, dtype=np.float64)
    S = px.shape[0]
    T = py.shape[1]
    p = np.full((S + 1, T + 1), np.nan)
    for s in range(s0, s1 + 1):
        for t in range(t0, t1 + 1):
            if s == s0 and t == t0:
                p[s, t] = 0.0
                continue
            a = -np.inf
            if s > s0:
                tt = t - 1 if modified else t
                if tt >= t0:
                    a = p[s - 1, tt] + px[s - 1, tt]
            b = -np.inf
            if t > t0:
                b = p[s, t - 1] + py[s, t - 1]
            p[s, t] = np.logaddexp(a, b)
    return p


def dp_torch(px, py, boundary, modified):
    """Differentiable float64 scores [B]; px/py are leaf tensors with grad."""
    B, S, _ = px.shape
    T = py.shape[2]
    scores = []
    ninf = torch.tensor(-math.inf, dtype=px.dtype)
    for b in range(B):
        s0, t0, s1, t1 = (0, 0, S, T) if boundary is None else [int(v) for v in boundary[b]]
        table = {}
        for s in range(s0, s1 + 1):
            for t in range(t0, t1 + 1):
                if s == s0 and t == t0:
                    table[(s, t)] = torch.zeros((), dtype=px.dtype)
                    continue
                a = ninf
                if s > s0:
                    tt = t - 1 if modified else t
                    if tt >= t0:
                        a = table[(s - 1, tt)] + px[b, s - 1, tt]
                c = ninf
                if t > t0:
                    c = table[(s, t - 1)] + py[b, s, t - 1]
                if torch.isinf(a) and torch.isinf(c):
                    table[(s, t)] = ninf
                elif torch.isinf(a):
                    table[(s, t)] = c
                elif torch.isinf(c):
                    table[(s, t)] = a
                else:
                    table[(s, t)] = torch.logaddexp(a, c)
        scores.append(table[(s1, t1)])
    return torch.stack(scores)


def log_binom(n, k):
    if k < 0 or k > n:
        return -math.inf
    return math.lgamma(n + 1) - math.lgamma(k + 1) - math.lgamma(n - k + 1)


def transducer_nll_bruteforce(logits_lsm, symbols, blank):
    """-log P(symbols) by enumerating alignments of a standard transducer.

    logits_lsm: [T][S+1][C] log-softmax outputs (nested lists / array), one
    utterance; the last frame must end with a blank.
    """
    lsm = np.asarray(logits_lsm, dtype=np.float64)
    T, S1, _ = lsm.shape
    S = S1 - 1
    total = -math.inf
    # a path is an interleaving of S symbols and T blanks ending with a blank
    for xs in itertools.combinations(range(S + T - 1), S):
        xs = set(xs)
        s = t = 0
        acc = 0.0
        for k in range(S + T - 1):
            if k in xs:
                acc += lsm[t, s, symbols[s]]
                s += 1
            else:
                acc += lsm[t, s, blank]
                t += 1
        acc += lsm[T - 1, S, blank]
        total = np.logaddexp(total, acc)
    return -float(total)
