"""Target and blank log-probs of every lattice cell, without materialising the log-softmax.

Drop-in for nemo/collections/asr/parts/k2/rnnt_logprobs_triton.py: `rnnt_logprobs(logits, targets,
blank_id, source_lengths=None, target_lengths=None)` returns `(target_scores, blank_scores)`, both
float32 `[B, T, U+1]`, zero outside each utterance and in the column that has no target
(:228-251); `RnntLogProbs` is the autograd Function behind it (:130-225).  The caller on the
reference side is GraphRnntLoss.forward (parts/k2/graph_transducer.py:517).

What differs from the reference: the forward leaves the row denominators in a small workspace
(4 bytes per cell) that the backward reuses, so the backward reads the logits once instead of
twice; pass `keep_forward_state=False` to get the reference's memory behaviour (nothing kept, the
backward recomputes).  bfloat16 / float16 logits are read natively, arithmetic is float32.
"""

import torch

from speech_amd import _native
from speech_amd.rnnt_loss.rnnt_pytorch import grads_like
from speech_amd.rnnt_loss.rnnt import _dtype_code, _labels_ptr, _ptr, _require_gpu, _stream, new_workspace

__all__ = ["RnntLogProbs", "rnnt_logprobs", "rnnt_logprobs_triton"]


def _lengths(lengths, fill, batch, device):
    if lengths is None:  # :150-158: every utterance spans the whole tensor
        return torch.full([batch], fill, dtype=torch.int64, device=device)
    return lengths.to(device=device, dtype=torch.int64).contiguous()


class RnntLogProbs(torch.autograd.Function):
    """log_softmax(logits)[..., targets] and log_softmax(logits)[..., blank_id] with autograd support."""

    @staticmethod
    def forward(ctx, logits, targets, blank_id, source_lengths, target_lengths, keep_forward_state=True):
        _require_gpu(logits, "rnnt_logprobs")
        assert logits.is_contiguous()  # :146: the logits are too large to copy silently
        if logits.dim() != 4:
            raise ValueError("logits must be [B, T, U+1, V]")
        B, T, U, V = logits.shape
        if targets.dim() != 2 or targets.shape[0] != B or targets.shape[1] != U - 1:
            raise ValueError(f"targets must be [B, U] = [{B}, {U - 1}], got {list(targets.shape)}")
        device = logits.device
        targets = targets.to(device=device, dtype=torch.int64).contiguous()
        source_lengths = _lengths(source_lengths, T, B, device)
        target_lengths = _lengths(target_lengths, U - 1, B, device)
        target_scores = torch.empty(B, T, U, dtype=torch.float32, device=device)
        blank_scores = torch.empty_like(target_scores)
        workspace = new_workspace(logits)
        with torch.cuda.device(device):
            status = _native.lib().mi_rnnt_logprobs_forward(
                _ptr(logits), _dtype_code(logits), _labels_ptr(targets), _ptr(source_lengths), _ptr(target_lengths),
                _ptr(target_scores), _ptr(blank_scores), B, T, U, V, int(blank_id), _ptr(workspace),
                workspace.numel(), _stream(device),
            )  # fmt: skip
        _native.check_status(status, "rnnt_logprobs forward")
        ctx.save_for_backward(logits, targets, source_lengths, target_lengths)
        ctx.blank_id = int(blank_id)
        ctx.workspace = workspace if keep_forward_state else None
        return target_scores, blank_scores

    @staticmethod
    def backward(ctx, grad_target_scores, grad_blank_scores):
        logits, targets, source_lengths, target_lengths = ctx.saved_tensors
        B, T, U, V = logits.shape
        device = logits.device
        workspace, have_state = ctx.workspace, 1
        if workspace is None:
            workspace, have_state = new_workspace(logits), 0
        grad_target_scores = grad_target_scores.to(torch.float32).contiguous()
        grad_blank_scores = grad_blank_scores.to(torch.float32).contiguous()
        grad_logits = grads_like(logits)  # every element is written, padded cells as zeros
        with torch.cuda.device(device):
            status = _native.lib().mi_rnnt_logprobs_backward(
                _ptr(logits), _dtype_code(logits), _labels_ptr(targets), _ptr(source_lengths), _ptr(target_lengths),
                _ptr(grad_target_scores), _ptr(grad_blank_scores), _ptr(grad_logits), have_state, B, T, U, V,
                ctx.blank_id, _ptr(workspace), workspace.numel(), _stream(device),
            )  # fmt: skip
        _native.check_status(status, "rnnt_logprobs backward")
        return grad_logits, None, None, None, None, None


def rnnt_logprobs(logits, targets, blank_id, source_lengths=None, target_lengths=None, keep_forward_state=True):
    """(target_scores, blank_scores), float32 [B, T, U+1], for logits [B, T, U+1, V] and targets [B, U]."""
    return RnntLogProbs.apply(logits, targets, blank_id, source_lengths, target_lengths, keep_forward_state)


def rnnt_logprobs_triton(logits, targets, blank_id, source_lengths=None, target_lengths=None):
    """The reference's name and signature for the same op (rnnt_logprobs_triton.py:228-251)."""
    return rnnt_logprobs(logits, targets, blank_id, source_lengths, target_lengths)
