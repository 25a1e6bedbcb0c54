"""GPU parity of the fused joint + multi-blank loss (mi_joint_multiblank_forward / _backward through
speech_amd.joint) against oracle.joint_rnnt_loss(..., big_blank_durations=...): the big blanks are ordinary outputs
of the joint's Linear layer at blank-1-i (rnnt_pytorch.py:442-510).  Tolerances as in tests/test_gpu_joint.py."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import MultiblankRNNTLossNumba
from speech_amd.joint import joint_multiblank_forward, joint_multiblank_loss

from gpu_utils import DEV

pytestmark = pytest.mark.gpu


def make_case(seed, B, T, U, H, V, NB):
    rng = np.random.RandomState(seed)
    f = torch.tensor(rng.randn(B, T, H), dtype=torch.bfloat16)
    g = torch.tensor(rng.randn(B, U, H), dtype=torch.bfloat16)
    W = torch.tensor(rng.randn(V, H) / np.sqrt(H), dtype=torch.float32)
    bias = torch.tensor(rng.randn(V) * 0.5, dtype=torch.float32)
    labels = rng.randint(0, V - 1 - NB, size=(B, U - 1))
    al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
    al[0], ll[-1] = T, U - 1
    return f, g, W, bias, labels, al, ll


def dev_ints(*arrays):
    return [torch.tensor(np.asarray(a), dtype=torch.int64, device=DEV) for a in arrays]


def check(seed, B, T, U, H, V, big_blanks, sigma=0.05, lam=0.0, clamp=0.0, blank=None, activation="relu"):
    NB = len(big_blanks)
    blank = V - 1 if blank is None else blank
    f, g, W, bias, labels, al, ll = make_case(seed, B, T, U, H, V, NB)
    labels = np.minimum(labels, max(blank - NB - 1, 0))
    gc = (np.random.RandomState(seed + 1000).rand(B) + 0.5).astype(np.float32)
    ref = oracle.joint_rnnt_loss(f.float().numpy(), g.float().numpy(), W.numpy(), bias.numpy(), labels, al, ll, blank,
                                 lam, clamp, gc, big_blank_durations=big_blanks, sigma=sigma, activation=activation)  # fmt: skip
    fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    Wd, bd = W.to(DEV).requires_grad_(True), bias.to(DEV).requires_grad_(True)
    lab, ald, lld = dev_ints(labels, al, ll)
    costs = joint_multiblank_loss(fd, gd, Wd, bd, lab, ald, lld, blank, big_blanks, sigma, lam, clamp,
                                  activation=activation)
    (costs * torch.tensor(gc, device=DEV)).sum().backward()
    torch.cuda.synchronize()
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref[0], rtol=1e-5)
    for name, x, want in zip(("d_f", "d_g", "d_weight", "d_bias"), (fd.grad, gd.grad, Wd.grad, bd.grad), ref[1:]):
        assert x.shape == want.shape, name
        err = np.abs(x.float().cpu().numpy() - want).max()
        assert err <= 2.0**-6 * np.abs(want).max() + 1e-7, (name, err, np.abs(want).max())
    # the big-blank rows of the weight gradient on their own
    rows = [blank - 1 - i for i in range(NB)]
    wd, want_d = Wd.grad[rows].float().cpu().numpy(), ref[3][rows]
    assert np.abs(wd - want_d).max() <= 2.0**-6 * np.abs(ref[3]).max() + 1e-7


@pytest.mark.parametrize("H", [256, 320, 384, 512, 640])
@pytest.mark.parametrize("V", [9, 34, 131, 1028])
def test_every_hidden_size_and_position_of_the_big_blanks(H, V):
    # V = 34: the big blanks cross a 32-row group (rows 30..32); 131: a 128-row block (127..129)
    check(V + H, 3, 9, 5, H, V, [2, 4, 8])


@pytest.mark.parametrize("big_blanks", [[2], [2, 4], [2, 3, 4, 5, 6, 7, 8, 9]])
def test_big_blank_sets_fastemit_clamp(big_blanks):
    check(len(big_blanks), 3, 12, 4, 640, 61, big_blanks, lam=0.01, clamp=0.1)


def test_blank_in_the_middle():
    check(7, 3, 9, 5, 512, 40, [2, 4], blank=20)


def test_forward_agrees_with_the_loss_module_on_materialised_logits():
    big_blanks, V = [2, 4, 8], 1028
    f, g, W, bias, labels, al, ll = make_case(6, 4, 30, 11, 640, V, len(big_blanks))
    lab, ald, lld = dev_ints(labels, al, ll)
    fd, gd, Wd, bd = f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV)
    fused = joint_multiblank_forward(fd, gd, Wd, bd, lab, ald, lld, V - 1, big_blanks, sigma=0.05)
    hidden = torch.relu(fd.unsqueeze(2) + gd.unsqueeze(1)).float()
    logits = hidden @ Wd.to(torch.bfloat16).float().t() + bd
    module = MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=big_blanks, reduction='none', sigma=0.05)
    unfused = module(logits.contiguous(), lab, ald, lld)
    np.testing.assert_allclose(fused.cpu().numpy(), unfused.float().cpu().numpy(), rtol=2e-5)


def test_rejects_bad_arguments():
    f, g, W, bias, labels, al, ll = make_case(8, 2, 4, 3, 256, 12, 2)
    lab, ald, lld = dev_ints(labels, al, ll)
    args = (f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV), lab, ald, lld)
    with pytest.raises(ValueError):
        joint_multiblank_forward(*args, 11, [])
    with pytest.raises(ValueError):
        joint_multiblank_forward(*args, 1, [2, 4])  # no room for two big blanks below blank = 1
    with pytest.raises(RuntimeError):
        joint_multiblank_forward(*args, 11, list(range(2, 11)))  # nine big blanks


def test_sigmoid_joint():
    check(5, 3, 8, 5, 384, 131, [2, 3], lam=0.01, activation="sigmoid")
