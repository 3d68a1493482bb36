"""Best-path alignment: same interface as ``i6_native_ops.fast_viterbi``
(i6_native_ops/fast_viterbi/__init__.py:23-47) on the MI355X library.

The extension module is built ahead of time by ``python -m i6_native_ops_amd.build``; there is no
import-time compilation and no CPU fallback.
"""
from typing import Tuple

import torch

from .._version import __version__  # noqa: F401  (fast_viterbi/__init__.py:8 of the reference)

try:
    from . import fast_viterbi_core as core
except ImportError as exc:  # pragma: no cover - depends on the build state
    raise ImportError(
        "i6_native_ops_amd.fast_viterbi needs the built extension fast_viterbi_core; "
        "run `python -m i6_native_ops_amd.build`"
    ) from exc

__all__ = ["align_viterbi", "core"]


def align_viterbi(
    log_probs: torch.FloatTensor,
    fsa: Tuple[int, torch.IntTensor, torch.FloatTensor, torch.IntTensor],
    seq_lens: torch.IntTensor,
) -> Tuple[torch.IntTensor, torch.FloatTensor]:
    """Find the best path with the Viterbi algorithm.

    :param log_probs: log probabilities of the emission model, shape (B, T, F)
    :param fsa: weighted finite state automaton as a tuple of
        * the number of states,
        * a (4, E) int tensor whose columns are origin state, target state, emission index and
          sequence index of an edge,
        * an (E,) float tensor of edge weights (added to the log probabilities),
        * a (2, B) int tensor of start states (row 0) and end states (row 1)
    :param seq_lens: (B,) int tensor of sequence lengths
    :return: (B, T) int tensor with the emission index of every frame of the best path and a
        (B,) tensor of its score
    """
    num_states, edge_tensor, weight_tensor, start_end_states = fsa
    if log_probs.dim() == 3 and log_probs.stride(2) != 1:
        log_probs = log_probs.contiguous()
    alignment, scores = core.fast_viterbi_batch_major(
        log_probs, edge_tensor, weight_tensor, start_end_states, seq_lens, num_states
    )
    return alignment, scores
