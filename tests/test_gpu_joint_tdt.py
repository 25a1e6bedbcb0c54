"""GPU parity of the fused joint + TDT loss (mi_joint_tdt_forward / mi_joint_tdt_backward through
speech_amd.joint) against oracle.joint_rnnt_loss(..., durations=...): the joint's Linear layer has V + D outputs, the
token logits followed by the duration logits (rnnt_pytorch.py:563-568).

Tolerances as for the RNNT variant (tests/test_gpu_joint.py): costs 1e-5 relative; every gradient tensor within 2^-6
of its own largest entry (the gradient of the logits and d hidden are bf16, as in autocast; the probabilities come from an
fp16 copy of the logits)."""

import random

import numpy as np
import pytest
import torch

import oracle
from speech_amd import TDTLossNumba
from speech_amd.joint import joint_dropout_mask, joint_rnnt_loss, joint_tdt_forward, joint_tdt_loss

from gpu_utils import DEV

pytestmark = pytest.mark.gpu


def make_case(seed, B, T, U, H, V, D, ragged=True):
    rng = np.random.RandomState(seed)
    f = torch.tensor(rng.randn(B, T, H), dtype=torch.bfloat16)
    g = torch.tensor(rng.randn(B, U, H), dtype=torch.bfloat16)
    W = torch.tensor(rng.randn(V + D, H) / np.sqrt(H), dtype=torch.float32)
    bias = torch.tensor(rng.randn(V + D) * 0.5, dtype=torch.float32)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    if ragged:
        al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
        al[0], ll[-1] = T, U - 1
    else:
        al, ll = np.full(B, T), np.full(B, U - 1)
    return f, g, W, bias, labels, al, ll


def dev_ints(*arrays):
    return [torch.tensor(np.asarray(a), dtype=torch.int64, device=DEV) for a in arrays]


def check(seed, B, T, U, H, V, durations, sigma=0.05, lam=0.0, clamp=0.0, ragged=True, bias_on=True,
          weight_dtype=torch.float32, dropout=0.0, activation="relu"):  # fmt: skip
    D = len(durations)
    f, g, W, bias, labels, al, ll = make_case(seed, B, T, U, H, V, D, ragged)
    gc = (np.random.RandomState(seed + 1000).rand(B) + 0.5).astype(np.float32)
    Wq = W.to(weight_dtype)
    bq = bias.to(weight_dtype) if bias_on else None
    rng_seed = 424242 + seed
    keep = joint_dropout_mask(B, T, U, H, dropout, rng_seed, DEV).cpu().numpy() if dropout else None
    ref = oracle.joint_rnnt_loss(f.float().numpy(), g.float().numpy(), Wq.float().numpy(),
                                 None if bq is None else bq.float().numpy(), labels, al, ll, V - 1, lam, clamp, gc,
                                 keep_mask=keep, dropout_p=dropout, durations=durations, sigma=sigma,
                                 activation=activation)  # fmt: skip
    fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    Wd = Wq.to(DEV).requires_grad_(True)
    bd = None if bq is None else bq.to(DEV).requires_grad_(True)
    lab, ald, lld = dev_ints(labels, al, ll)
    costs = joint_tdt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, durations, sigma, lam, clamp, dropout=dropout,
                           seed=rng_seed, activation=activation)  # fmt: skip
    (costs * torch.tensor(gc, device=DEV)).sum().backward()
    torch.cuda.synchronize()
    assert costs.dtype == torch.float32 and costs.shape == (B,)
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref[0], rtol=1e-5)
    got = [fd.grad, gd.grad, Wd.grad] + ([] if bd is None else [bd.grad])
    for name, x, want in zip(("d_f", "d_g", "d_weight", "d_bias"), got, ref[1:]):
        assert x.shape == want.shape, name
        err = np.abs(x.float().cpu().numpy() - want).max()
        assert err <= 2.0**-6 * np.abs(want).max() + 1e-7, (name, err, np.abs(want).max())
    # the duration rows of the weight gradient on their own: they are small beside the token rows
    wd, want_d = Wd.grad[V:].float().cpu().numpy(), ref[3][V:]
    assert np.abs(wd - want_d).max() <= 2.0**-6 * np.abs(want_d).max() + 1e-7
    assert Wd.grad.dtype == weight_dtype
    return costs


@pytest.mark.parametrize("H", [256, 320, 384, 512, 640])
@pytest.mark.parametrize("V", [3, 30, 126, 128, 1025])
def test_every_hidden_size_and_position_of_the_duration_rows(H, V):
    # V = 30: the duration rows cross a 32-row group; 126: a 128-row block; 128: they start a block of their own
    check(V + H, 3, 7, 5, H, V, [0, 1, 2, 3, 4])


@pytest.mark.parametrize("durations", [[1], [0, 1], [1, 2], [0, 1, 2, 4], [0, 1, 2, 3, 4, 5, 6, 7]])
def test_duration_sets(durations):
    check(len(durations), 3, 9, 4, 640, 61, durations)


def test_fastemit_clamp_no_bias_bf16_weights_full_lengths():
    check(1, 3, 9, 6, 640, 130, [0, 1, 2], lam=0.01, clamp=0.05)
    check(2, 2, 6, 4, 512, 300, [0, 1, 2, 3], ragged=False, bias_on=False, weight_dtype=torch.bfloat16)


def test_dropout():
    check(3, 3, 8, 5, 640, 77, [0, 1, 2, 3, 4], lam=0.01, dropout=0.3)


def test_many_tiles_and_utterances():
    check(4, 5, 60, 13, 640, 257, [0, 1, 2, 3, 4])
    check(5, 70, 3, 2, 384, 19, [0, 1])


def test_forward_agrees_with_the_loss_module_on_materialised_logits():
    """The unfused pipeline of the reference: joint tensor first, then TDTLossNumba on it."""
    durations, V = [0, 1, 2, 3, 4], 1025
    f, g, W, bias, labels, al, ll = make_case(6, 4, 30, 11, 640, V, len(durations))
    lab, ald, lld = dev_ints(labels, al, ll)
    fd, gd, Wd, bd = f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV)
    fused = joint_tdt_forward(fd, gd, Wd, bd, lab, ald, lld, V - 1, durations, sigma=0.05)
    hidden = torch.relu(fd.unsqueeze(2) + gd.unsqueeze(1)).float()
    logits = hidden @ Wd.to(torch.bfloat16).float().t() + bd
    unfused = TDTLossNumba(blank=V - 1, durations=durations, reduction='none', sigma=0.05)(logits.contiguous(), lab, ald, lld)
    np.testing.assert_allclose(fused.cpu().numpy(), unfused.float().cpu().numpy(), rtol=2e-5)


def test_omega_one_is_the_rnnt_loss_on_the_token_rows():
    durations, V, H = [0, 1, 2], 40, 512
    f, g, W, bias, labels, al, ll = make_case(7, 3, 6, 5, H, V, len(durations))
    lab, ald, lld = dev_ints(labels, al, ll)

    def run(fn):
        fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
        Wd, bd = W.to(DEV).requires_grad_(True), bias.to(DEV).requires_grad_(True)
        costs = fn(fd, gd, Wd, bd)
        costs.sum().backward()
        return costs.detach(), fd.grad, gd.grad, Wd.grad, bd.grad

    random.seed(0)
    a = run(lambda fd, gd, Wd, bd: joint_tdt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, durations, 0.05, omega=1.0))
    b = run(lambda fd, gd, Wd, bd: joint_rnnt_loss(fd, gd, Wd[:V], bd[:V], lab, ald, lld, V - 1))
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    assert torch.all(a[3][V:] == 0) and torch.all(a[4][V:] == 0)


def test_rejects_bad_duration_arguments():
    f, g, W, bias, labels, al, ll = make_case(8, 2, 4, 3, 256, 10, 3)
    lab, ald, lld = dev_ints(labels, al, ll)
    args = (f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV), lab, ald, lld)
    with pytest.raises(ValueError):
        joint_tdt_forward(*args, 9, [])
    with pytest.raises(ValueError):
        joint_tdt_forward(*args, 10, [0, 1, 2])  # blank inside the duration rows
    with pytest.raises(RuntimeError):
        joint_tdt_forward(*args, 3, list(range(9)))  # more than 8 durations
    with pytest.raises(RuntimeError):
        joint_tdt_forward(*args, 9, [0, 2, 3])  # no duration 1 among the first two (gpu_rnnt_kernel.py:1137-1148)


@pytest.mark.parametrize("tdt", [False, True])
def test_backward_agrees_with_autograd_of_the_unfused_pipeline(tdt):
    """Several tiles per utterance AND nine row blocks of vocabulary (too large for the per-cell oracle loops): the
    reference's pipeline in float32 on the same GPU -- joint tensor from the bf16-rounded operands, loss module,
    torch autograd -- against the fused op, gradients at the bf16 tolerance of the other tests."""
    durations = [0, 1, 2, 3, 4] if tdt else []
    V, H, B, T, U = 1025, 640, 3, 40, 15
    f, g, W, bias, labels, al, ll = make_case(11, B, T, U, H, V, len(durations))
    lab, ald, lld = dev_ints(labels, al, ll)
    gc = torch.tensor([0.5, 1.0, 1.5], device=DEV)

    def leaves():
        return (f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True),
                W.to(torch.bfloat16).float().to(DEV).requires_grad_(True), bias.to(DEV).requires_grad_(True))  # fmt: skip

    fd, gd, Wd, bd = leaves()
    if tdt:
        costs = joint_tdt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, durations, 0.05, 0.01)
    else:
        costs = joint_rnnt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, 0.01)
    (costs * gc).sum().backward()
    fr, gr, Wr, br = leaves()
    hidden = torch.relu(fr.unsqueeze(2) + gr.unsqueeze(1)).float()
    logits = hidden @ Wr.t() + br
    if tdt:
        module = TDTLossNumba(blank=V - 1, durations=durations, reduction='none', sigma=0.05, fastemit_lambda=0.01)
    else:
        from speech_amd import RNNTLossNumba

        module = RNNTLossNumba(blank=V - 1, reduction='none', fastemit_lambda=0.01)
    ref = module(logits, lab, ald, lld).float()
    (ref * gc).sum().backward()
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref.detach().cpu().numpy(), rtol=2e-5)
    for name, x, want in (("d_f", fd.grad, fr.grad), ("d_g", gd.grad, gr.grad), ("d_weight", Wd.grad, Wr.grad),
                          ("d_bias", bd.grad, br.grad)):  # fmt: skip
        err = (x.float() - want.float()).abs().max().item()
        assert err <= 2.0**-6 * want.float().abs().max().item() + 1e-7, (name, err)


@pytest.mark.parametrize("tdt", [False, True])
def test_fused_sub_batches_give_the_same_costs_and_gradients(tdt):
    """fused_batch_size (the reference's sub-batch loop, modules/rnnt.py:1527-1587): utterances do not interact, so the
    costs are the same numbers and the gradients differ by the order of a few bf16-rounded partial sums at most."""
    durations = [0, 1, 2] if tdt else []
    V, H, B, T, U = 50, 320, 7, 12, 6
    f, g, W, bias, labels, al, ll = make_case(12, B, T, U, H, V, len(durations))
    lab, ald, lld = dev_ints(labels, al, ll)

    def run(fbs):
        fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
        Wd, bd = W.to(DEV).requires_grad_(True), bias.to(DEV).requires_grad_(True)
        if tdt:
            costs = joint_tdt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, durations, 0.05, fused_batch_size=fbs)
        else:
            costs = joint_rnnt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, fused_batch_size=fbs)
        costs.sum().backward()
        return costs.detach(), fd.grad.float(), gd.grad.float(), Wd.grad, bd.grad

    whole, parts = run(None), run(3)
    assert parts[0].shape == (B,) and torch.equal(whole[0], parts[0])
    for x, y in zip(whole[1:], parts[1:]):
        assert (x - y).abs().max().item() <= 2.0**-7 * x.abs().max().item()
    with pytest.raises(ValueError):
        run(-1)


@pytest.mark.parametrize("activation", ["tanh", "sigmoid"])
def test_tanh_and_sigmoid_joints_with_dropout(activation):
    """modules/rnnt.py:1762-1776: activation, then Dropout, then the Linear layer."""
    check(77, 3, 9, 5, 640, 130, [0, 1, 2], lam=0.01, dropout=0.2, activation=activation)
