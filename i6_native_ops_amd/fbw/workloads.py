"""Seeded synthetic FBW workloads (host side, NumPy only).

The five named workloads are the benchmark configurations: tiny HMM, monophone
hybrid HMM, CART-state full-sum (headline), CTC topology and long-form CART.
Everything is drawn from ``numpy.random.default_rng(seed)`` (PCG64) on the
host, so the same seed gives bit-identical inputs on any machine.

The automata follow the convention of the reference's own fixture
(test/fbw.py:28-32): emissions sit on edges, every edge consumes one frame, a
sequence has one start and one end state, and states are numbered contiguously
across the batch.  The tuple layout is the one ``fbw_loss`` documents
(i6_native_ops/fbw/__init__.py:56-62).
"""
from dataclasses import dataclass
from typing import List, Optional, Tuple

import numpy as np


@dataclass
class Workload:
    name: str
    am_scores: Optional[np.ndarray]   # float32 [T,B,F], -log softmax (None if with_am=False)
    edges: np.ndarray                 # int32 [4,E]: from, to, emission_idx, sequence_idx
    weights: np.ndarray               # float32 [E]
    start_end_states: np.ndarray      # int32 [2,B]
    seq_lens: np.ndarray              # int32 [B]
    n_states: int
    T: int
    B: int
    F: int

    @property
    def E(self) -> int:
        return int(self.edges.shape[1])

    def edges_per_seq(self) -> np.ndarray:
        return np.bincount(self.edges[3], minlength=self.B)

    def algorithmic_bytes(self) -> int:
        """Bytes one loss+grad call has to move at element granularity, every datum once:
        dense (T,B,F) write + one gathered score per edge per valid frame + the edge
        list + the (T,B) loss + start/end/seq_len."""
        valid = np.clip(self.seq_lens.astype(np.int64), 0, self.T)
        valid = np.where(self.seq_lens.astype(np.int64) > self.T, 0, valid)
        gather = int((valid * self.edges_per_seq().astype(np.int64)).sum())
        return 4 * self.T * self.B * self.F + 4 * gather + 20 * self.E + 4 * self.T * self.B + 12 * self.B

    def seq_frames(self) -> int:
        return int(np.clip(self.seq_lens, 0, self.T).sum())


class _Automaton:
    """Edge list of one sequence with local state ids."""

    def __init__(self):
        self.frm: List[int] = []
        self.to: List[int] = []
        self.emis: List[int] = []
        self.w: List[float] = []
        self.n_states = 0
        self.start = 0
        self.end = 0

    def new_state(self) -> int:
        self.n_states += 1
        return self.n_states - 1

    def edge(self, f: int, t: int, e: int, w: float):
        self.frm.append(f)
        self.to.append(t)
        self.emis.append(int(e))
        self.w.append(float(w))


def _hmm_chain(emis: List[int], loop_w, fwd_w, rng=None, sil_after=None, sil_emis=0, sil_in_w=None) -> _Automaton:
    """Left-to-right HMM: state i emits ``emis[i]`` on its loop and on its exit edge
    (emission = source state's label, as in test/fbw.py:28-32); one non-emitting
    terminal state.  ``sil_after[i]`` inserts a skippable silence state after state i.
    ``loop_w`` / ``fwd_w`` are callables returning a weight."""
    a = _Automaton()
    ids = [a.new_state() for _ in emis]
    sil_ids = {}
    if sil_after is not None:
        for i, flag in enumerate(sil_after):
            if flag:
                sil_ids[i] = a.new_state()
    term = a.new_state()
    for i, s in enumerate(ids):
        nxt = ids[i + 1] if i + 1 < len(ids) else term
        a.edge(s, s, emis[i], loop_w())
        a.edge(s, nxt, emis[i], fwd_w())
        if i in sil_ids:
            q = sil_ids[i]
            a.edge(s, q, emis[i], sil_in_w() if sil_in_w is not None else fwd_w())
            a.edge(q, q, sil_emis, loop_w())
            a.edge(q, nxt, sil_emis, fwd_w())
    a.start, a.end = ids[0], term
    return a


def _ctc(labels: List[int], blank: int = 0) -> _Automaton:
    """CTC topology with emissions on the *target* state.  A non-emitting virtual
    start feeds blank_0 and label_1; the two accepting states (last label, last
    blank) are merged into a single terminal state X that receives a copy of every
    edge entering either of them, so X can only be occupied after the last frame."""
    a = _Automaton()
    v = a.new_state()
    sym = [blank]
    for l in labels:
        sym += [int(l), blank]
    st = [a.new_state() for _ in sym]
    x = a.new_state()
    n = len(st)
    accepting = {n - 1, n - 2} if n >= 2 else {n - 1}

    def add(f, ti):
        a.edge(f, st[ti], sym[ti], 0.0)
        if ti in accepting:
            a.edge(f, x, sym[ti], 0.0)

    add(v, 0)
    if n > 1:
        add(v, 1)
    for i in range(n):
        add(st[i], i)
        if i + 1 < n:
            add(st[i], i + 1)
        if i + 2 < n and sym[i] != blank and sym[i + 2] != sym[i]:
            add(st[i], i + 2)
    a.start, a.end = v, x
    return a


def _assemble(name, autos: List[_Automaton], seq_lens, T, B, F, rng, sigma, with_am, shuffle_edges) -> Workload:
    frm, to, emis, seq, w = [], [], [], [], []
    starts, ends = [], []
    off = 0
    for b, a in enumerate(autos):
        frm += [f + off for f in a.frm]
        to += [t + off for t in a.to]
        emis += a.emis
        seq += [b] * len(a.frm)
        w += a.w
        starts.append(a.start + off)
        ends.append(a.end + off)
        off += a.n_states
    edges = np.array([frm, to, emis, seq], dtype=np.int32).reshape(4, -1)
    weights = np.array(w, dtype=np.float32)
    if shuffle_edges:
        perm = rng.permutation(edges.shape[1])
        edges = np.ascontiguousarray(edges[:, perm])
        weights = np.ascontiguousarray(weights[perm])
    am = make_am_scores(rng, T, B, F, sigma) if with_am else None
    return Workload(name, am, edges, weights, np.array([starts, ends], dtype=np.int32),
                    np.asarray(seq_lens, dtype=np.int32), off, T, B, F)


def make_am_scores(rng, T: int, B: int, F: int, sigma: float) -> np.ndarray:
    """-log_softmax of N(0, sigma) logits; softmax evaluated in float64, result float32."""
    am = np.empty((T, B, F), dtype=np.float32)
    step = max(1, (1 << 24) // max(1, B * F))
    for t0 in range(0, T, step):
        t1 = min(T, t0 + step)
        x = rng.standard_normal((t1 - t0, B, F), dtype=np.float32).astype(np.float64) * sigma
        m = x.max(axis=-1, keepdims=True)
        lse = m + np.log(np.exp(x - m).sum(axis=-1, keepdims=True))
        am[t0:t1] = (lse - x).astype(np.float32)
    return am


WORKLOADS = ("tiny", "monophone", "cart", "ctc", "longform")
_SHAPES = {
    "tiny": (50, 2, 10, 1.0),
    "monophone": (500, 32, 264, 2.0),
    "cart": (1000, 32, 12001, 3.0),
    "ctc": (200, 256, 5001, 2.0),
    "longform": (4000, 8, 12001, 3.0),
}


def make_workload(name: str, seed: Optional[int] = None, T: Optional[int] = None, B: Optional[int] = None,
                  F: Optional[int] = None, with_am: bool = True, shuffle_edges: bool = False,
                  n_labels: Optional[Tuple[int, int]] = None) -> Workload:
    """Builds one of the named workloads.  ``T``/``B``/``F``/``n_labels`` shrink it for
    tests; with the defaults and ``seed=None`` (-> 1000 + index) it is the benchmark case."""
    idx = WORKLOADS.index(name)
    T0, B0, F0, sigma = _SHAPES[name]
    T, B, F = T or T0, B or B0, F or F0
    rng = np.random.default_rng(1000 + idx + 1 if seed is None else seed)
    scale = T / T0
    autos: List[_Automaton] = []

    def n_lab(lo, hi):
        if n_labels is not None:
            lo, hi = n_labels
        else:
            lo, hi = max(1, int(lo * scale)), max(1, int(hi * scale))
        return int(rng.integers(lo, hi + 1))

    if name == "tiny":
        for _ in range(B):
            labels = rng.integers(0, F, size=n_lab(5, 5))
            emis = [int((l * 3 + s) % F) for l in labels for s in range(3)]
            autos.append(_hmm_chain(emis, lambda: 0.0, lambda: 0.0))
        seq_lens = [T, max(1, (T * 4) // 5)] + [T] * (B - 2) if B >= 2 else [T]
        seq_lens = seq_lens[:B]
    elif name == "monophone":
        n_phones = max(1, F // 3)
        w = float(-np.log(0.5))
        for _ in range(B):
            phones = rng.integers(0, n_phones, size=n_lab(40, 60))
            emis = [int(p * 3 + s) for p in phones for s in range(3)]
            sil = [False] * len(emis)
            flags = rng.random(len(phones)) < 0.5
            for i in range(len(phones) - 1):
                sil[i * 3 + 2] = bool(flags[i])
            autos.append(_hmm_chain(emis, lambda: w, lambda: w, sil_after=sil, sil_emis=F - 1))
        seq_lens = rng.integers(int(0.8 * T), T + 1, size=B)
    elif name in ("cart", "longform"):
        lo, hi = (100, 150) if name == "cart" else (400, 600)
        wdraw = lambda: float(-np.log(rng.uniform(0.3, 0.7)))
        for _ in range(B):
            n = n_lab(lo, hi)
            emis = [int(e) for e in rng.integers(0, F, size=3 * n)]
            sil = None
            sil_w = None
            if name == "longform":
                flags = rng.random(n) < 0.3
                sil = [False] * len(emis)
                for i in range(n - 1):
                    sil[i * 3 + 2] = bool(flags[i])
                sil_w = lambda: float(-np.log(0.2))
            autos.append(_hmm_chain(emis, wdraw, wdraw, sil_after=sil, sil_emis=F - 1, sil_in_w=sil_w))
        lo_t = int(0.8 * T) if name == "cart" else int(0.5 * T)
        seq_lens = rng.integers(lo_t, T + 1, size=B)
    elif name == "ctc":
        for _ in range(B):
            labels = rng.integers(1, F, size=n_lab(20, 60))
            autos.append(_ctc([int(l) for l in labels], blank=0))
        seq_lens = rng.integers(int(0.75 * T), T + 1, size=B)
    else:
        raise ValueError(name)
    return _assemble(name, autos, seq_lens, T, B, F, rng, sigma, with_am, shuffle_edges)
