"""Shared helpers of the test-suite: the reference's own fixture, a brute-force
path enumerator and small random automata."""
import itertools
import json
import os

import numpy as np


def golden(name):
    """One of the reference's own test vectors, kept as data in tests/golden/reference_fixtures.json."""
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_fixtures.json")) as f:
        return json.load(f)[name]


def _golden_arrays(name, sign):
    g = golden(name)
    p = np.array(g["probabilities"], dtype=np.float32)
    am = (sign * np.log(p))[:, None, :].astype(np.float32)      # [T,B,F]
    edges = np.array(g["edges"], dtype=np.int32).T.copy()
    weights = np.array(g["weights"], dtype=np.float32)
    start_end = np.array(g["start_end_states"], dtype=np.int32)
    return am, edges, weights, start_end, np.array(g["seq_lens"], dtype=np.int32), int(g["num_states"])


def reference_fixture(seq_len=5):
    """The one FBW fixture the reference holds (test/fbw.py:9-41): B=1, T=5, F=2,
    two states, three edges, all weights 1; scores are -log p."""
    am, edges, weights, start_end, seq_lens, n = _golden_arrays("fbw", -1.0)
    seq_lens[:] = seq_len
    return am, edges, weights, start_end, seq_lens, n


def reference_viterbi_fixture():
    """test/fast_viterbi.py:9-35: the same automaton with scores log p, and the alignment the
    reference's test expects."""
    return _golden_arrays("fast_viterbi", 1.0), np.array(golden("fast_viterbi")["expected"]["alignment"], dtype=np.int32)


def brute_force(am, edges, weights, start_end, seq_lens, n_states):
    """Enumerates every accepting path.  Returns (loss [T,B], posterior [T,B,F]) in
    float64 with the reference's conventions: loss 0 and posterior 0 on frames
    t >= seq_len, and for sequences without any accepting path."""
    T, B, F = am.shape
    am = am.astype(np.float64)
    loss = np.zeros((T, B))
    post = np.zeros((T, B, F))
    E = edges.shape[1]
    for b in range(B):
        L = int(seq_lens[b])
        if L < 1 or L > T:
            continue
        out_edges = {}
        for e in range(E):
            if edges[3, e] == b:
                out_edges.setdefault(int(edges[0, e]), []).append(e)
        total = 0.0
        acc = np.zeros((T, F))
        stack = [(int(start_end[0, b]), 0, 0.0, [])]
        while stack:
            s, t, sc, path = stack.pop()
            if t == L:
                if s == int(start_end[1, b]):
                    p = np.exp(-sc)
                    total += p
                    for tt, e in enumerate(path):
                        acc[tt, edges[2, e]] += p
                continue
            for e in out_edges.get(s, []):
                stack.append((int(edges[1, e]), t + 1, sc + float(weights[e]) + am[t, b, edges[2, e]], path + [e]))
        if total > 0:
            loss[:L, b] = -np.log(total)
            post[:L, b] = acc[:L] / total
    return loss, post


def random_fsa(rng, B, F, max_states=4, max_edges=8, T=5):
    """Small arbitrary automata: shared emission ids, parallel edges, unreachable
    and dead-end states, random weights, edges of all sequences interleaved."""
    frm, to, emis, seq, w = [], [], [], [], []
    starts, ends = [], []
    off = 0
    for b in range(B):
        ns = int(rng.integers(1, max_states + 1))
        ne = int(rng.integers(1, max_edges + 1))
        for _ in range(ne):
            frm.append(off + int(rng.integers(0, ns)))
            to.append(off + int(rng.integers(0, ns)))
            emis.append(int(rng.integers(0, F)))
            seq.append(b)
            w.append(float(rng.uniform(-0.5, 2.0)))
        starts.append(off + int(rng.integers(0, ns)))
        ends.append(off + int(rng.integers(0, ns)))
        off += ns
    perm = rng.permutation(len(frm))
    edges = np.array([frm, to, emis, seq], dtype=np.int32)[:, perm].copy()
    weights = np.array(w, dtype=np.float32)[perm].copy()
    am = rng.uniform(0.1, 4.0, size=(T, B, F)).astype(np.float32)
    seq_lens = rng.integers(1, T + 1, size=B).astype(np.int32)
    return am, edges, weights, np.array([starts, ends], dtype=np.int32), seq_lens, off


def posterior(out):
    """exp(-out): what FastBaumWelchLoss.backward returns (fbw/__init__.py:40-44)."""
    return np.exp(-out.astype(np.float64))


def spread_state_ids(edges, start_end, n_states, how="permute", seed=5):
    """The same automata under other state ids: "stride" multiplies every id by 11 (each sequence keeps a
    range of its own, eleven times as wide), "permute" draws the ids at random from a range three times as
    large (the ranges of all sequences overlap)."""
    if how == "stride":
        new_id = np.arange(n_states, dtype=np.int64) * 11 + 3
        total = n_states * 11 + 3
    else:
        total = n_states * 3
        new_id = np.random.default_rng(seed).permutation(total)[:n_states]
    out = edges.copy()
    out[0] = new_id[edges[0]]
    out[1] = new_id[edges[1]]
    return out, new_id[start_end].astype(np.int32), int(total)
