"""Automaton tuples for ``fbw_loss`` / ``align_viterbi`` built on the GPU.

The reference leaves the tuple ``(num_states, edges (4, E), weights (E,), start_end_states (2, B))``
to its callers (i6_native_ops/fbw/__init__.py:56-62).  These helpers build it on the device from
label tensors for the two usual topologies, through the C ABI of libi6fbw.so
(``i6fbw_build_ctc_fsa``, ``i6fbw_build_hmm_fsa``).  The edge tensors come back at a capacity that
always suffices; the unused tail consists of padding edges (sequence index -1) that the kernels
skip, so nothing is copied to the host and nothing synchronises.
"""
from typing import Optional, Tuple

import torch

from . import cabi

Fsa = Tuple[int, torch.Tensor, torch.Tensor, torch.Tensor]


def _check(labels: torch.Tensor, lens: torch.Tensor):
    if not (labels.is_cuda and lens.is_cuda):
        raise RuntimeError("labels and lengths must be CUDA tensors")
    if labels.dtype != torch.int32 or lens.dtype != torch.int32:
        raise RuntimeError("labels and lengths must be int32")
    if labels.dim() != 2 or lens.dim() != 1 or lens.shape[0] != labels.shape[0]:
        raise RuntimeError("labels must have shape (B, Lmax), lengths (B,)")
    if labels.shape[1] > 0 and labels.stride(1) != 1:
        labels = labels.contiguous()
    return labels, lens.contiguous()


def ctc_fsa(targets: torch.Tensor, target_lens: torch.Tensor, blank: int = 0, return_totals: bool = False):
    """CTC topology: with it ``fbw_loss(log_probs, ctc_fsa(...), seq_lens)[0]`` equals
    ``torch.nn.functional.ctc_loss(..., reduction="none")``.

    :param targets: (B, Lmax) int32 labels, rows padded arbitrarily
    :param target_lens: (B,) int32 number of labels per row
    :return: (state bound, edges (4, capacity) int32, weights (capacity,) float32, start_end_states (2, B) int32)
        and, if asked, a device tensor [edges produced, states]
    """
    targets, target_lens = _check(targets, target_lens)
    B, Lmax = targets.shape
    cap, n_states, scratch_bytes = cabi.ctc_fsa_bounds(B, Lmax)
    dev = targets.device
    with torch.cuda.device(dev):
        edges = torch.empty((4, cap), dtype=torch.int32, device=dev)
        weights = torch.empty((cap,), dtype=torch.float32, device=dev)
        start_end = torch.empty((2, B), dtype=torch.int32, device=dev)
        totals = torch.empty((2,), dtype=torch.int32, device=dev)
        scratch = torch.empty((scratch_bytes,), dtype=torch.uint8, device=dev)
        cabi.build_ctc_fsa(targets.data_ptr(), targets.stride(0), target_lens.data_ptr(), B, Lmax, int(blank), edges.data_ptr(),
                           edges.stride(0), cap, weights.data_ptr(), start_end.data_ptr(), start_end.stride(0),
                           totals.data_ptr(), scratch.data_ptr(), torch.cuda.current_stream().cuda_stream)
    fsa = (n_states, edges, weights, start_end)
    return (fsa, totals) if return_totals else fsa


def hmm_fsa(labels: torch.Tensor, label_lens: torch.Tensor, states_per_label: int = 3, loop_weight: float = 0.0,
            forward_weight: float = 0.0, emission_table: Optional[torch.Tensor] = None, return_totals: bool = False):
    """Left-to-right HMM chain: ``states_per_label`` states per label, each with a loop and an edge
    to the next state, both emitting ``emission_table[label * states_per_label + k]`` (that index
    itself without a table); weights are in -log space for ``fbw_loss``.

    :param labels: (B, Lmax) int32, rows padded arbitrarily
    :param label_lens: (B,) int32
    :param emission_table: optional int32 tensor mapping (label, state) to an emission index
    """
    labels, label_lens = _check(labels, label_lens)
    B, Lmax = labels.shape
    cap = max(1, 2 * B * Lmax * states_per_label)
    n_states = B * (Lmax * states_per_label + 1)
    dev = labels.device
    if emission_table is not None:
        if not emission_table.is_cuda or emission_table.dtype != torch.int32:
            raise RuntimeError("emission_table must be an int32 CUDA tensor")
        emission_table = emission_table.contiguous()
    with torch.cuda.device(dev):
        edges = torch.empty((4, cap), dtype=torch.int32, device=dev)
        weights = torch.empty((cap,), dtype=torch.float32, device=dev)
        start_end = torch.empty((2, B), dtype=torch.int32, device=dev)
        totals = torch.empty((2,), dtype=torch.int32, device=dev)
        cabi.build_hmm_fsa(labels.data_ptr(), labels.stride(0), label_lens.data_ptr(), B, Lmax, int(states_per_label),
                           emission_table.data_ptr() if emission_table is not None else None, float(loop_weight),
                           float(forward_weight), edges.data_ptr(), edges.stride(0), cap, weights.data_ptr(),
                           start_end.data_ptr(), start_end.stride(0), totals.data_ptr(),
                           torch.cuda.current_stream().cuda_stream)
    fsa = (n_states, edges, weights, start_end)
    return (fsa, totals) if return_totals else fsa
