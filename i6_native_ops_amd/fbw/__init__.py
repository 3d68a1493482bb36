"""Full-sum forward-backward (FBW) loss on MI355X.

Same public surface as ``i6_native_ops.fbw`` (i6_native_ops/fbw/__init__.py:27-68):
``fbw_loss``, ``FastBaumWelchLoss`` and the extension module ``core`` (``fbw_core``) with
``fbw`` and ``DebugOptions``.  The extension is built ahead of time by
``i6_native_ops_amd/build.py``; nothing is compiled at import, and there is no CPU or eager
fallback: without the built HIP library the import fails.

Problems only the device can see (an index out of range) do not make a call wait for the device:
they are raised by a later call or by ``check_status()``; ``set_status_mode("sync")`` makes every
call wait and raise for itself (the reference has undefined behaviour there).
"""
from typing import Tuple

import torch  # noqa: F401  (libtorch must be loaded before the extension)

from .._version import __version__  # noqa: F401  (fbw/__init__.py:8 of the reference)

try:
    from . import fbw_core as core
except ImportError as exc:  # pragma: no cover
    raise ImportError(
        "i6_native_ops_amd.fbw: the HIP extension fbw_core / libi6fbw.so is not built. "
        "Run `python -m i6_native_ops_amd.build` (needs hipcc and PyTorch-ROCm)."
    ) from exc


class FastBaumWelchLoss(torch.autograd.Function):
    """Counterpart of the reference's autograd function (fbw/__init__.py:27-44).

    forward returns the (T, B) tensor in which every valid frame of sequence b holds the total
    negative log-likelihood of b (padded frames hold 0); backward ignores the incoming gradient
    and returns the state posteriors (T, B, F) as the gradient w.r.t. ``am_scores``, exactly as
    the reference does.  The posteriors come straight from the kernel instead of ``exp(-out)``.
    """

    @staticmethod
    def forward(ctx, am_scores, fsa, seq_lens):
        num_states, edge_tensor, weight_tensor, start_end_states = fsa
        posterior, loss = core.fbw_posterior(
            am_scores, edge_tensor, weight_tensor, start_end_states, seq_lens, int(num_states)
        )
        ctx.save_for_backward(posterior)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        return ctx.saved_tensors[0], None, None


class _FusedFbwLoss(torch.autograd.Function):
    """fbw_loss without the wrapper's dense passes: the kernels read ``log_probs`` (B, T, F) in place
    (sign flip and strides inside the gather) and write the gradient w.r.t. ``log_probs``, minus
    the posteriors, in (B, T, F).  Same values as FastBaumWelchLoss behind the reference's
    neg/transpose/contiguous chain (fbw/__init__.py:40-44,66), including the ignored grad_loss."""

    @staticmethod
    def forward(ctx, log_probs, fsa, seq_lens):
        num_states, edge_tensor, weight_tensor, start_end_states = fsa
        if log_probs.stride(-1) != 1:
            log_probs = log_probs.contiguous()
        grad, loss = core.fbw_fused(log_probs, edge_tensor, weight_tensor, start_end_states, seq_lens,
                                    int(num_states))
        ctx.save_for_backward(grad)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        return ctx.saved_tensors[0], None, None


def fbw_loss(
    log_probs: torch.FloatTensor,
    fsa: Tuple[int, torch.IntTensor, torch.FloatTensor, torch.IntTensor],
    seq_lens: torch.IntTensor,
) -> torch.FloatTensor:
    """Negative log-likelihood of an emission model given an HMM automaton; the gradient w.r.t.
    ``log_probs`` (minus the state posteriors) is back-propagated automatically.

    :param log_probs: log probabilities of the emission model, [B, T, F]
    :param fsa: (number of states, int32 (4, E) edges with rows from / to / emission idx /
        sequence idx, float32 (E,) edge weights, int32 (2, B) start and end states)
    :param seq_lens: int32 (B,) sequence lengths
    :return: (T, B) tensor; entry (t, b) is the loss of sequence b for t < seq_lens[b], else 0
        (the reference's docstring says (B,), its code returns (T, B): fbw/__init__.py:32-38)
    """
    return _FusedFbwLoss.apply(log_probs, fsa, seq_lens)


def fbw_loss_unfused(log_probs, fsa, seq_lens):
    """The reference's literal wrapper (fbw/__init__.py:66-67): explicit negation and transposition in
    front of FastBaumWelchLoss.  Kept for comparison; fbw_loss gives the same values faster."""
    neg_log_probs = log_probs.neg().transpose(0, 1).contiguous()  # [T, B, F]
    return FastBaumWelchLoss.apply(neg_log_probs, fsa, seq_lens)


set_status_mode = core.set_status_mode
check_status = core.check_status

__all__ = ["fbw_loss", "fbw_loss_unfused", "FastBaumWelchLoss", "core", "set_status_mode", "check_status"]
