"""Pins the multi-blank transducer oracle.  The reference holds no vector for this loss (its test
compares two of its own implementations on random input, test_rnnt_pytorch.py:510-541), so the
pins are: the RNNT golden vectors for the degenerate case without big blanks, brute-force path
enumeration, torch autograd of an alpha-only recursion, and invariants."""

import numpy as np
import pytest

import oracle
from oracle import transducer_numpy as onp

from helpers import multiblank_autograd, multiblank_bruteforce_ll

IMPLS = ["numpy", "c"]


def run_mb(impl, acts, labels, act_lens, label_lens, blank, durs, sigma, lam=0.0, clamp=0.0, dtype=np.float64):
    if impl == "numpy":
        return onp.multiblank_loss(acts, labels, act_lens, label_lens, blank, durs, sigma, lam, clamp, dtype=dtype)
    return oracle.multiblank_loss(acts, labels, act_lens, label_lens, blank, durs, sigma, lam, clamp, dtype=dtype)


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name", ["small", "small_blank_last", "medium"])
def test_without_big_blanks_it_is_the_rnnt_loss(golden, impl, name):
    """No big blank and sigma = 0: the reference's RNNT vectors (cost + full gradient) must come out."""
    g = golden[name]
    acts = np.array(g["acts"], dtype=np.float64)
    costs, grads, ex = run_mb(impl, acts, g["labels"], g["act_lens"], g["label_lens"], g["blank"], [], 0.0)
    assert np.allclose(costs, g["costs"], rtol=1e-6, atol=g.get("atol", 1e-8))
    assert np.allclose(grads, np.array(g["grads"]), atol=max(g.get("atol", 1e-8), 1e-6))
    assert np.allclose(ex["ll_forward"], ex["ll_backward"], atol=1e-10)


@pytest.mark.parametrize("impl", IMPLS)
def test_sigma_shifts_the_cost_by_the_path_length_when_there_is_no_big_blank(impl):
    """Without big blanks every path has exactly T + U - 1 arcs, so sigma adds (T+U-1)*sigma to the cost
    and leaves the gradient alone."""
    rng = np.random.RandomState(3)
    T, U, V = 5, 4, 6
    x = rng.randn(1, T, U, V)
    labels = rng.randint(0, V - 1, size=(1, U - 1))
    c0, g0, _ = run_mb(impl, x, labels, [T], [U - 1], V - 1, [], 0.0)
    c1, g1, _ = run_mb(impl, x, labels, [T], [U - 1], V - 1, [], 0.3)
    assert abs(c1[0] - c0[0] - 0.3 * (T + U - 1)) < 1e-10
    assert np.abs(g1 - g0).max() < 1e-12


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("durs", [[2], [2, 3], [2, 4, 8], [3], [5, 2]])
def test_bruteforce_and_autograd(impl, durs):
    rng = np.random.RandomState(23)
    sigma = 0.1
    NB = len(durs)
    for T, U, Vtok in [(1, 1, 2), (2, 1, 2), (4, 1, 3), (4, 2, 3), (5, 3, 3), (6, 3, 2), (9, 2, 2)]:
        V = Vtok + NB + 1
        blank = V - 1
        x = rng.randn(1, T, U, V)
        labels = rng.randint(0, Vtok, size=(1, max(U - 1, 0)))
        ll_bf = multiblank_bruteforce_ll(x[0], labels[0], blank, durs, sigma)
        costs, grads, ex = run_mb(impl, x, labels, [T], [U - 1], blank, durs, sigma)
        assert abs(-costs[0] - ll_bf) < 1e-10
        nll, g = multiblank_autograd(x[0], labels[0], blank, durs, sigma)
        assert abs(nll - costs[0]) < 1e-10
        assert np.abs(g - grads[0]).max() < 1e-10
        assert abs(ex["ll_forward"][0] - ex["ll_backward"][0]) < 1e-10
        assert np.abs(grads[0].sum(-1)).max() < 1e-10  # every row of the logits-gradient sums to zero


@pytest.mark.parametrize("impl", IMPLS)
def test_blank_in_the_middle_of_the_alphabet(impl):
    """The standard blank need not be last: big blank i is at blank-1-i wherever blank is."""
    rng = np.random.RandomState(5)
    T, U, V = 5, 3, 8
    durs, blank = [2, 3], 4  # big blanks at 3 and 2, tokens 0,1,5,6,7
    x = rng.randn(1, T, U, V)
    labels = np.array([[6, 0]])
    costs, grads, _ = run_mb(impl, x, labels, [T], [U - 1], blank, durs, 0.05)
    assert abs(-costs[0] - multiblank_bruteforce_ll(x[0], labels[0], blank, durs, 0.05)) < 1e-10
    nll, g = multiblank_autograd(x[0], labels[0], blank, durs, 0.05)
    assert np.abs(g - grads[0]).max() < 1e-10


@pytest.mark.parametrize("impl", IMPLS)
def test_fastemit_and_clamp(impl):
    """FastEmit: derived only (no reference vector): label-arc log-prob gradient x (1+lambda) through the
    softmax Jacobian, cost x (1+lambda).  Clamp: elementwise clip of that gradient."""
    rng = np.random.RandomState(8)
    T, U, Vtok, durs, sigma, lam = 6, 4, 4, [2, 4], 0.1, 0.25
    V = Vtok + len(durs) + 1
    x = rng.randn(1, T, U, V)
    labels = rng.randint(0, Vtok, size=(1, U - 1))
    costs, grads, _ = run_mb(impl, x, labels, [T], [U - 1], V - 1, durs, sigma, lam=lam)
    nll, g = multiblank_autograd(x[0], labels[0], V - 1, durs, sigma, lam=lam)
    assert abs(nll - costs[0]) < 1e-10
    assert np.abs(g - grads[0]).max() < 1e-10
    _, gc, _ = run_mb(impl, x, labels, [T], [U - 1], V - 1, durs, sigma, lam=lam, clamp=0.05)
    assert np.abs(gc - np.clip(g, -0.05, 0.05)[None]).max() < 1e-10


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_batch_with_variable_lengths_numpy_equals_c_and_sliced_utterances(dtype):
    rng = np.random.RandomState(31)
    B, T, U, Vtok, durs, sigma = 3, 7, 4, 5, [2, 4], 0.1
    V = Vtok + len(durs) + 1
    x = rng.randn(B, T, U, V)
    labels = rng.randint(0, Vtok, size=(B, U - 1))
    act_lens, label_lens = [7, 4, 6], [3, 1, 0]
    cn, gn, _ = onp.multiblank_loss(x, labels, act_lens, label_lens, V - 1, durs, sigma, 0.01, 0.2, dtype=dtype)
    cc, gc, _ = oracle.multiblank_loss(x, labels, act_lens, label_lens, V - 1, durs, sigma, 0.01, 0.2, dtype=dtype)
    tol = 1e-12 if dtype == np.float64 else 2e-5
    assert np.allclose(cn, cc, rtol=tol, atol=tol) and np.abs(gn - gc).max() < tol
    for b in range(B):
        Tb, Ub = act_lens[b], label_lens[b] + 1
        c1, g1, _ = oracle.multiblank_loss(
            x[b : b + 1, :Tb, :Ub], labels[b : b + 1, : Ub - 1], [Tb], [Ub - 1], V - 1, durs, sigma, 0.01, 0.2, dtype=dtype
        )
        assert np.allclose(c1[0], cc[b], rtol=tol) and np.abs(g1[0] - gc[b, :Tb, :Ub]).max() < tol
        pad = gc[b].copy()
        pad[:Tb, :Ub] = 0
        assert np.all(pad == 0)
