"""Shared plumbing of the GPU parity tests (imported only by tests marked `gpu`)."""

import numpy as np
import torch

DEV = "cuda:0"


def to_dev(labels, act_lens, label_lens):
    return (
        torch.as_tensor(np.asarray(labels), dtype=torch.int64, device=DEV).contiguous(),
        torch.as_tensor(np.asarray(act_lens), dtype=torch.int64, device=DEV),
        torch.as_tensor(np.asarray(label_lens), dtype=torch.int64, device=DEV),
    )


def call_loss(fn, acts, labels, act_lens=None, label_lens=None, dtype=torch.float32):
    """The reference's wrap_and_call (tests/collections/asr/numba/rnnt_loss/test_rnnt_pytorch.py:44-73)
    with optional explicit lengths: sum the costs, backward, return (costs, grad) as numpy."""
    acts_t = torch.as_tensor(np.asarray(acts), dtype=dtype).to(DEV).requires_grad_(True)
    B, T, U = acts_t.shape[:3]
    labels = np.asarray(labels, dtype=np.int64).reshape(B, -1)
    if act_lens is None:
        act_lens = [T] * B
    if label_lens is None:
        label_lens = [labels.shape[1]] * B
    lab, al, ll = to_dev(labels, act_lens, label_lens)
    costs = fn(acts_t, lab, al, ll)
    costs.sum().backward()
    torch.cuda.synchronize()
    return costs.detach().float().cpu().numpy(), acts_t.grad.float().cpu().numpy()


def make_lengths(rng, B, T, U, t_lo, u_lo):
    """Uniform lengths with one utterance forced to T and one to U-1 so that the shape check passes."""
    act_lens = rng.randint(t_lo, T + 1, size=B)
    label_lens = rng.randint(u_lo, U, size=B)
    act_lens[rng.randint(B)] = T
    label_lens[rng.randint(B)] = U - 1
    return act_lens.astype(np.int64), label_lens.astype(np.int64)
