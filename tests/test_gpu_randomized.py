"""Seeded random sweeps of the GPU path against the oracle: shapes, lengths, vocabulary sizes across every row-length
class, blank positions, dtypes, reductions, FastEmit, clamp, sigma, duration sets (with and without duration 0, so
utterances without any alignment occur) and big-blank sets.  Costs 1e-5 relative; gradients 1e-4 absolute for float32
(relative to the largest entry where the sentinel arithmetic of an impossible alignment makes them huge), one 16-bit
rounding step for 16-bit logits."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba

from gpu_utils import DEV

pytestmark = pytest.mark.gpu


def run(fn, x, labels, act_lens, label_lens):
    a = x.to(DEV).requires_grad_(True)
    B = x.shape[0]
    c = fn(a, torch.tensor(labels, dtype=torch.int64, device=DEV).reshape(B, -1), torch.tensor(act_lens, device=DEV),
           torch.tensor(label_lens, device=DEV))  # fmt: skip
    c.sum().backward()
    torch.cuda.synchronize()
    return c.detach().float().cpu().numpy(), a.grad.float().cpu().numpy()


def lengths(rng, B, T, U):
    al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
    al[rng.randint(B)], ll[rng.randint(B)] = T, U - 1
    return al, ll


def check(costs, grads, c_ref, g_ref, dtype, float32_costs=False):
    # RNNT costs are float32 whatever the logits' dtype (rnnt_pytorch.py:60); TDT costs take the dtype of the logits
    tol = 1e-4 if dtype == torch.float32 else 2.0**-7
    np.testing.assert_allclose(costs, c_ref, rtol=1e-5 if dtype == torch.float32 or float32_costs else 2.0**-7)
    assert np.abs(grads - g_ref).max() <= tol * max(1.0, np.abs(g_ref).max())


VOCABS = [2, 3, 5, 17, 64, 65, 129, 255, 256, 257, 511, 513, 1025, 2049, 4097, 8193, 9000, 16385, 20011]


@pytest.mark.parametrize("block", range(3))
def test_rnnt(block):
    rng = np.random.RandomState(4242 + block)
    for it in range(block * 19, block * 19 + 19):
        B, T, U, V = int(rng.randint(1, 5)), int(rng.randint(1, 20)), int(rng.randint(1, 10)), VOCABS[it % len(VOCABS)]
        dtype = [torch.float32, torch.bfloat16, torch.float16][it % 3]
        lam, clamp = float(rng.choice([0.0, 0.01])), float(rng.choice([0.0, 0.2]))
        blank = int(rng.choice([0, V - 1, rng.randint(0, V)]))
        x = torch.tensor(rng.randn(B, T, U, V) * rng.choice([1.0, 5.0]), dtype=dtype)
        labels = rng.randint(0, V, size=(B, U - 1))
        al, ll = lengths(rng, B, T, U)
        reduction = ['none', 'sum', 'mean'][it % 3]
        c_ref, g_ref, _ = oracle.rnnt_loss(x.float().numpy(), labels, al, ll, blank, lam, clamp)
        if reduction != 'none':
            c_ref = c_ref.sum(keepdims=True)
        if reduction == 'mean':
            c_ref, g_ref = c_ref / B, g_ref / B
        fn = RNNTLossNumba(blank=blank, reduction=reduction, fastemit_lambda=lam, clamp=clamp if clamp > 0 else -1)
        check(*run(fn, x, labels, al, ll), c_ref, g_ref, dtype, True)


DURATION_SETS = [[0, 1], [1], [1, 2], [0, 1, 2], [1, 2, 4], [0, 1, 3, 6], [0, 1, 2, 3, 4], [1, 3],
                 [0, 1, 2, 3, 4, 5, 6, 7], [1, 2, 3, 4, 5, 9], [0, 1, 2, 3, 4, 5, 6, 7, 8, 9]]  # fmt: skip


@pytest.mark.parametrize("block", range(3))
def test_tdt(block):
    rng = np.random.RandomState(777 + block)
    for it in range(block * 22, block * 22 + 22):
        B, T, U = int(rng.randint(1, 5)), int(rng.randint(1, 24)), int(rng.randint(1, 12))
        V = int(rng.randint(2, 60)) if it % 4 else [1025, 2500, 5001][it % 3]
        durs = DURATION_SETS[it % len(DURATION_SETS)]
        dtype = torch.float32 if durs[0] != 0 else [torch.float32, torch.bfloat16, torch.float16][it % 3]
        sigma, lam = float(rng.choice([0.0, 0.05])), float(rng.choice([0.0, 0.01]))
        clamp = float(rng.choice([0.0, 0.3]))
        x = torch.tensor(rng.randn(B, T, U, V + len(durs)) * rng.choice([1.0, 4.0]), dtype=dtype)
        labels = rng.randint(0, V - 1, size=(B, U - 1))
        al, ll = lengths(rng, B, T, U)
        c_ref, g_ref, _ = oracle.tdt_loss(x.float().numpy(), labels, al, ll, V - 1, durs, sigma, lam, clamp)
        fn = TDTLossNumba(blank=V - 1, durations=durs, reduction='none', sigma=sigma, fastemit_lambda=lam,
                          clamp=clamp if clamp > 0 else -1)  # fmt: skip
        check(*run(fn, x, labels, al, ll), c_ref, g_ref, dtype)


BIG_BLANK_SETS = [[], [2], [2, 4], [2, 4, 8], [3, 5, 7, 9, 11], [2, 3, 4, 5, 6, 7, 8, 9], [1, 2], [20]]


@pytest.mark.parametrize("block", range(2))
def test_multiblank(block):
    rng = np.random.RandomState(31 + block)
    for it in range(block * 16, block * 16 + 16):
        B, T, U, Vt = int(rng.randint(1, 5)), int(rng.randint(1, 24)), int(rng.randint(1, 12)), int(rng.randint(1, 40))
        durs = BIG_BLANK_SETS[it % len(BIG_BLANK_SETS)]
        V = Vt + len(durs) + 1
        sigma, lam = float(rng.choice([0.0, 0.05])), float(rng.choice([0.0, 0.01]))
        x = torch.tensor(rng.randn(B, T, U, V) * rng.choice([1.0, 4.0]), dtype=torch.float32)
        labels = rng.randint(0, Vt, size=(B, U - 1))
        al, ll = lengths(rng, B, T, U)
        c_ref, g_ref, _ = oracle.multiblank_loss(x.numpy(), labels, al, ll, V - 1, durs, sigma, lam, 0.0)
        fn = MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=durs, reduction='none', sigma=sigma,
                                     fastemit_lambda=lam)  # fmt: skip
        check(*run(fn, x, labels, al, ll), c_ref, g_ref, torch.float32)
