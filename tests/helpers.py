"""Shared helpers of the test-suite: the reference's own fixture, a brute-force
path enumerator and small random automata."""
import itertools

import numpy as np


def reference_fixture(seq_len=5):
    """The one FBW fixture the reference holds (test/fbw.py:9-41): B=1, T=5, F=2,
    two states, three edges, all weights 1."""
    p = np.array([[0.9, 0.1], [0.9, 0.1], [0.4, 0.6], [0.1, 0.9], [0.1, 0.9]], dtype=np.float32)
    am = (-np.log(p))[:, None, :].astype(np.float32)            # [T,B,F]
    edges = np.array([[0, 0, 0, 0], [0, 1, 0, 0], [1, 1, 1, 0]], dtype=np.int32).T.copy()
    weights = np.ones(3, dtype=np.float32)
    start_end = np.array([[0], [1]], dtype=np.int32)
    seq_lens = np.array([seq_len], dtype=np.int32)
    return am, edges, weights, start_end, seq_lens, 2


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
