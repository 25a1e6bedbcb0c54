"""Pins oracle.joint_rnnt_loss (joint network + RNNT loss under bf16-autocast arithmetic).

The reference holds no vector for joint + loss together; its joint is torch's own relu / Linear
(nemo/collections/asr/modules/rnnt.py:1707-1724, :1759-1777).  So the oracle is checked against those
library routines and their autograd, in float64, on inputs that are exact in bf16; the loss itself is
oracle.rnnt_loss, pinned by the reference's golden vectors elsewhere.
"""

import numpy as np
import pytest
import torch

import oracle
from oracle.transducer_numpy import bf16_round

from helpers import joint_autograd


def test_bf16_round_matches_torch():
    rng = np.random.RandomState(0)
    x = np.concatenate([rng.randn(4000) * 10.0 ** rng.randint(-6, 6, size=4000), [0.0, -0.0, 1.0, 65280.0, 3.0e38]])
    # exact ties: halfway between two bf16 neighbours
    ties = (np.arange(1, 200, dtype=np.uint32) << 16 | 0x8000) + 0x3F800000
    x = np.concatenate([x.astype(np.float32), ties.view(np.float32)])
    expect = torch.tensor(x, dtype=torch.float32).to(torch.bfloat16).double().numpy()
    np.testing.assert_array_equal(bf16_round(x), expect)


@pytest.mark.parametrize("shape", [(1, 2, 2, 8, 3), (2, 3, 4, 16, 7), (2, 4, 3, 32, 11)])
def test_against_torch_autograd(shape):
    B, T, U, H, V = shape
    rng = np.random.RandomState(B * 100 + T)
    f, g = bf16_round(rng.randn(B, T, H)), bf16_round(rng.randn(B, U, H))
    w = bf16_round(rng.randn(V, H) / np.sqrt(H))
    bias = bf16_round(rng.randn(V))
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    gc = rng.rand(B) + 0.5
    costs, d_f, d_g, d_w, d_b = oracle.joint_rnnt_loss(f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc)
    ref = joint_autograd(f, g, w, bias, labels, V - 1, gc)
    for got, want in zip((costs, d_f, d_g, d_w, d_b), ref):
        np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("activation", ["tanh", "sigmoid"])
def test_tanh_and_sigmoid_joints_against_torch_autograd(activation):
    """The reference's joint may use tanh or sigmoid (modules/rnnt.py:1762-1770).  Exactly: torch's own activation with
    its output rounded to bf16 and the slope taken at the rounded output.  Loosely (1 %, the size of a bf16 rounding
    step on every slope): plain float64 autograd that knows nothing of that convention -- a wrong derivative or a
    slope taken at the wrong place would be off by tens of percent."""
    B, T, U, H, V = 2, 3, 4, 16, 7
    rng = np.random.RandomState(31)
    f, g = bf16_round(rng.randn(B, T, H)), bf16_round(rng.randn(B, U, H))
    w, bias = bf16_round(rng.randn(V, H) / np.sqrt(H)), bf16_round(rng.randn(V))
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    gc = rng.rand(B) + 0.5
    got = oracle.joint_rnnt_loss(f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc, activation=activation)
    ref = joint_autograd(f, g, w, bias, labels, V - 1, gc, activation=activation)
    for a, b in zip(got, ref):
        np.testing.assert_allclose(a, b, rtol=1e-9, atol=1e-11)
    loose = joint_autograd(f, g, w, bias, labels, V - 1, gc, activation=activation, rounded_activation=False)
    np.testing.assert_allclose(got[0], loose[0], rtol=2e-3)
    for a, b in zip(got[1:], loose[1:]):
        assert np.abs(a - b).max() <= 2e-2 * np.abs(b).max()
    with pytest.raises(ValueError):
        oracle.joint_rnnt_loss(f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, activation="gelu")


def test_ragged_lengths_are_the_trimmed_problems():
    B, T, U, H, V = 3, 5, 4, 16, 9
    rng = np.random.RandomState(7)
    f, g = rng.randn(B, T, H), rng.randn(B, U, H)
    w, bias = rng.randn(V, H) / 4, rng.randn(V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    al, ll = np.array([5, 2, 4]), np.array([1, 3, 0])
    costs, d_f, d_g, d_w, d_b = oracle.joint_rnnt_loss(f, g, w, bias, labels, al, ll, V - 1, fastemit_lambda=0.01)
    sum_w, sum_b = np.zeros_like(d_w), np.zeros_like(d_b)
    for b in range(B):
        Tb, Ub = al[b], ll[b] + 1
        c1, f1, g1, w1, b1 = oracle.joint_rnnt_loss(
            f[b : b + 1, :Tb], g[b : b + 1, :Ub], w, bias, labels[b : b + 1, : Ub - 1], [Tb], [Ub - 1], V - 1,
            fastemit_lambda=0.01,
        )
        np.testing.assert_allclose(costs[b], c1[0], rtol=1e-12)
        np.testing.assert_allclose(d_f[b, :Tb], f1[0], atol=1e-12)
        np.testing.assert_allclose(d_g[b, :Ub], g1[0], atol=1e-12)
        assert np.all(d_f[b, Tb:] == 0) and np.all(d_g[b, Ub:] == 0)
        sum_w += w1
        sum_b += b1
    np.testing.assert_allclose(d_w, sum_w, atol=1e-11)
    np.testing.assert_allclose(d_b, sum_b, atol=1e-11)


def test_dropout_against_torch_autograd():
    B, T, U, H, V = 2, 3, 3, 16, 7
    rng = np.random.RandomState(9)
    f, g = bf16_round(rng.randn(B, T, H)), bf16_round(rng.randn(B, U, H))
    w, bias = bf16_round(rng.randn(V, H) / 4), bf16_round(rng.randn(V))
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    keep = rng.rand(B, T, U, H) >= 0.3
    gc = rng.rand(B) + 0.5
    got = oracle.joint_rnnt_loss(f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc, keep_mask=keep, dropout_p=0.3)
    ref = joint_autograd(f, g, w, bias, labels, V - 1, gc, keep_mask=keep, dropout_p=0.3)
    for a, b in zip(got, ref):
        np.testing.assert_allclose(a, b, rtol=1e-9, atol=1e-11)
    # a mask of ones with p = 0 is no dropout at all
    plain = oracle.joint_rnnt_loss(f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc)
    ones = oracle.joint_rnnt_loss(f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc,
                                  keep_mask=np.ones((B, T, U, H), dtype=bool), dropout_p=0.0)  # fmt: skip
    for a, b in zip(plain, ones):
        np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("durations", [[0, 1, 2], [1, 2], [0, 1, 2, 3, 4]])
def test_tdt_variant_against_torch_autograd(durations):
    """With `durations` the Linear layer has V + D outputs and the loss is the TDT one: checked against torch autograd
    of relu / Linear fed with the logits-gradient of an independent alpha-only TDT recursion (helpers.tdt_autograd).
    f + g is exact in bf16 here (multiples of 1/8 below 4), so no rounding enters."""
    from helpers import tdt_autograd

    B, T, U, H, V, D, sigma = 2, 4, 3, 16, 6, len(durations), 0.05
    rng = np.random.RandomState(D)
    f, g = rng.randint(-16, 17, size=(B, T, H)) / 8.0, rng.randint(-16, 17, size=(B, U, H)) / 8.0
    w, bias = bf16_round(rng.randn(V + D, H) / 4), bf16_round(rng.randn(V + D))
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    gc = rng.rand(B) + 0.5
    costs, d_f, d_g, d_w, d_b = oracle.joint_rnnt_loss(
        f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc, durations=durations, sigma=sigma
    )
    ft, gt = torch.tensor(f, requires_grad=True), torch.tensor(g, requires_grad=True)
    wt, bt = torch.tensor(w, requires_grad=True), torch.tensor(bias, requires_grad=True)
    logits = torch.nn.functional.linear(torch.relu(ft[:, :, None, :] + gt[:, None, :, :]), wt, bt)
    d_logits = []
    for b in range(B):
        nll, gl = tdt_autograd(logits[b].detach().numpy(), labels[b], V - 1, durations, sigma)
        np.testing.assert_allclose(costs[b], nll, rtol=1e-10)
        d_logits.append(gl * gc[b])
    logits.backward(torch.tensor(np.stack(d_logits)))
    for got, want in zip((d_f, d_g, d_w, d_b), (ft.grad, gt.grad, wt.grad, bt.grad)):
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("big_blanks", [[2], [2, 4], [2, 3, 5]])
def test_multiblank_variant_against_torch_autograd(big_blanks):
    """With `big_blank_durations` the loss is the multi-blank one (big blanks at outputs blank-1-i of the same
    softmax): checked as the TDT variant above, with helpers.multiblank_autograd as the independent recursion."""
    from helpers import multiblank_autograd

    B, T, U, H, sigma = 2, 5, 3, 16, 0.05
    V = 5 + len(big_blanks) + 1
    rng = np.random.RandomState(len(big_blanks))
    f, g = rng.randint(-16, 17, size=(B, T, H)) / 8.0, rng.randint(-16, 17, size=(B, U, H)) / 8.0
    w, bias = bf16_round(rng.randn(V, H) / 4), bf16_round(rng.randn(V))
    labels = rng.randint(0, 5, size=(B, U - 1))
    gc = rng.rand(B) + 0.5
    costs, d_f, d_g, d_w, d_b = oracle.joint_rnnt_loss(
        f, g, w, bias, labels, [T] * B, [U - 1] * B, V - 1, grad_costs=gc, big_blank_durations=big_blanks, sigma=sigma
    )
    ft, gt = torch.tensor(f, requires_grad=True), torch.tensor(g, requires_grad=True)
    wt, bt = torch.tensor(w, requires_grad=True), torch.tensor(bias, requires_grad=True)
    logits = torch.nn.functional.linear(torch.relu(ft[:, :, None, :] + gt[:, None, :, :]), wt, bt)
    d_logits = []
    for b in range(B):
        nll, gl = multiblank_autograd(logits[b].detach().numpy(), labels[b], V - 1, big_blanks, sigma)
        np.testing.assert_allclose(costs[b], nll, rtol=1e-10)
        d_logits.append(gl * gc[b])
    logits.backward(torch.tensor(np.stack(d_logits)))
    for got, want in zip((d_f, d_g, d_w, d_b), (ft.grad, gt.grad, wt.grad, bt.grad)):
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-9, atol=1e-11)
