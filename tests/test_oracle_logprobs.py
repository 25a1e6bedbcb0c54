"""Pins the oracle of the compact log-prob op (oracle.rnnt_logprobs / rnnt_logprobs_grad).

The reference holds no stored vector for this op: its test compares the kernel with a torch
etalon, log_softmax + gather (tests/collections/asr/k2/test_graph_transducer.py:295-336,
parts/k2/rnnt_logprobs.py:19-48).  The same etalon is used here, in float64, and the backward is
checked against torch autograd through it -- a library routine and its derivative, not the
oracle's own formulas.
"""

import numpy as np
import pytest
import torch

import oracle


def etalon(logits, targets, blank):
    """log_softmax + gather with library calls only (the shape of rnnt_logprobs_torch, :19-48)."""
    B = logits.shape[0]
    log_probs = torch.log_softmax(logits, dim=-1)
    blank_scores = log_probs[..., blank]
    ids = torch.cat([targets, torch.zeros(B, 1, dtype=targets.dtype)], dim=-1)
    target_scores = torch.gather(log_probs, -1, ids[:, None, :, None].expand(*log_probs.shape[:-1], 1)).squeeze(-1)
    mask = torch.ones_like(target_scores)
    mask[:, :, -1] = 0.0
    return target_scores * mask, blank_scores


def case(seed, B, T, U, V, ragged):
    rng = np.random.RandomState(seed)
    logits = rng.randn(B, T, U, V) * 2.0
    targets = rng.randint(0, V - 1, size=(B, U - 1))
    if ragged:
        src = rng.randint(1, T + 1, size=B)
        tgt = rng.randint(0, U, size=B)
        src[0], tgt[-1] = T, U - 1
    else:
        src = tgt = None
    return logits, targets, src, tgt


@pytest.mark.parametrize("shape", [(1, 1, 1, 2), (2, 3, 4, 5), (3, 7, 5, 33), (2, 4, 6, 257)])
def test_forward_is_log_softmax_gather(shape):
    B, T, U, V = shape
    logits, targets, _, _ = case(1, B, T, U, V, False)
    ts, bs = oracle.rnnt_logprobs(logits, targets, V - 1)
    ts_ref, bs_ref = etalon(torch.tensor(logits), torch.tensor(targets), V - 1)
    np.testing.assert_allclose(ts, ts_ref.numpy(), atol=1e-12)
    np.testing.assert_allclose(bs, bs_ref.numpy(), atol=1e-12)
    assert np.all(ts[:, :, -1] == 0.0)


@pytest.mark.parametrize("blank_first", [True, False])
def test_backward_is_autograd_of_the_etalon(blank_first):
    B, T, U, V = 3, 6, 5, 17
    rng = np.random.RandomState(2)
    logits = rng.randn(B, T, U, V)
    blank = 0 if blank_first else V - 1
    targets = rng.randint(1, V - 1, size=(B, U - 1))  # never the blank id
    gt, gb = rng.rand(B, T, U), rng.rand(B, T, U)
    x = torch.tensor(logits, requires_grad=True)
    ts, bs = etalon(x, torch.tensor(targets), blank)
    (torch.tensor(gt) * ts + torch.tensor(gb) * bs).sum().backward()
    got = oracle.rnnt_logprobs_grad(logits, targets, blank, gt, gb)
    np.testing.assert_allclose(got, x.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(got.sum(-1), 0.0, atol=1e-12)  # a log-softmax gradient row sums to gb+gt-(gb+gt) = 0


def test_ragged_lengths_mask_rows_and_targets():
    B, T, U, V = 4, 6, 5, 9
    logits, targets, src, tgt = case(3, B, T, U, V, True)
    ts, bs = oracle.rnnt_logprobs(logits, targets, V - 1, src, tgt)
    ts_full, bs_full = oracle.rnnt_logprobs(logits, targets, V - 1)
    gt, gb = np.random.RandomState(4).rand(2, B, T, U)
    g = oracle.rnnt_logprobs_grad(logits, targets, V - 1, gt, gb, src, tgt)
    for b in range(B):
        Tb, Ub = src[b], tgt[b] + 1
        np.testing.assert_array_equal(bs[b, :Tb, :Ub], bs_full[b, :Tb, :Ub])
        np.testing.assert_array_equal(ts[b, :Tb, : Ub - 1], ts_full[b, :Tb, : Ub - 1])
        assert np.all(ts[b, :, Ub - 1 :] == 0) and np.all(ts[b, Tb:] == 0)
        assert np.all(bs[b, :, Ub:] == 0) and np.all(bs[b, Tb:] == 0)
        assert np.all(g[b, Tb:] == 0) and np.all(g[b, :, Ub:] == 0)
        # inside the utterance: the full-tensor gradient of the trimmed problem
        sub = oracle.rnnt_logprobs_grad(
            logits[b : b + 1, :Tb, :Ub], targets[b : b + 1, : Ub - 1], V - 1, gt[b : b + 1, :Tb, :Ub], gb[b : b + 1, :Tb, :Ub]
        )
        np.testing.assert_allclose(g[b, :Tb, :Ub], sub[0], atol=1e-14)


def test_target_equal_to_blank_keeps_only_the_target_term():
    """rnnt_logprobs_triton.py:120-122: the second `where` overwrites the first, so the blank gradient's
    direct term is dropped at that one logit (autograd of the etalon would add both)."""
    B, T, U, V = 1, 2, 3, 4
    rng = np.random.RandomState(5)
    logits = rng.randn(B, T, U, V)
    blank = 2
    targets = np.array([[2, 1]])
    gt, gb = rng.rand(B, T, U), rng.rand(B, T, U)
    x = torch.tensor(logits, requires_grad=True)
    ts, bs = etalon(x, torch.tensor(targets), blank)
    (torch.tensor(gt) * ts + torch.tensor(gb) * bs).sum().backward()
    expect = x.grad.numpy().copy()
    expect[:, :, 0, blank] -= gb[:, :, 0]
    np.testing.assert_allclose(oracle.rnnt_logprobs_grad(logits, targets, blank, gt, gb), expect, atol=1e-12)
