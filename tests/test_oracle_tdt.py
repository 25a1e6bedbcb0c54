"""Pins the TDT oracle against the reference's fixed vector, brute-force path
enumeration, torch autograd and closed-form special cases."""

import numpy as np
import pytest
from scipy.special import log_softmax, logsumexp

import oracle
from oracle import transducer_numpy as onp

from helpers import tdt_autograd, tdt_bruteforce_ll

IMPLS = ["numpy", "c"]


def run_tdt(impl, acts, labels, act_lens, label_lens, blank, durations, sigma, lam=0.0, clamp=0.0, dtype=np.float64):
    if impl == "numpy":
        return onp.tdt_loss(acts, labels, act_lens, label_lens, blank, durations, sigma, lam, clamp, dtype=dtype)
    return oracle.tdt_loss(acts, labels, act_lens, label_lens, blank, durations, sigma, lam, clamp, dtype=dtype)


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_golden_fixed_vector(golden, impl, dtype):
    # tests/collections/asr/numba/rnnt_loss/test_rnnt_pytorch.py:593-625
    g = golden["tdt_fixed"]
    acts = np.zeros(g["shape"])
    costs, grads, ex = run_tdt(
        impl, acts, g["labels"], g["act_lens"], g["label_lens"], g["blank"], g["durations"], g["sigma"], dtype=dtype
    )
    assert np.allclose(costs, g["costs"], rtol=1e-6)  # the reference's own tolerance
    assert np.allclose(grads, np.array(g["grads"]), atol=1e-7, rtol=2e-6)  # far inside its rtol=1e-2
    assert np.allclose(ex["ll_forward"], ex["ll_backward"], atol=1e-6)


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("durations", [[0, 1, 2], [0, 1, 2, 3, 4], [1, 2, 3], [0, 1], [1], [0, 1, 3]])
def test_bruteforce_and_autograd(impl, durations):
    rng = np.random.RandomState(17)
    D = len(durations)
    sigma = 0.05
    for T, U, V in [(1, 1, 3), (3, 1, 3), (4, 2, 3), (4, 3, 4), (5, 3, 3)]:
        blank = V - 1
        x = rng.randn(1, T, U, V + D)
        labels = rng.randint(0, V - 1, size=(1, max(U - 1, 0)))
        ll_bf = tdt_bruteforce_ll(x[0], labels[0], blank, durations, sigma)
        if ll_bf == -np.inf:
            continue  # no complete path (e.g. U > 1 without a duration that can stay in frame)
        costs, grads, ex = run_tdt(impl, x, labels, [T], [U - 1], blank, durations, sigma)
        # the finite -10000 sentinel contributes exp(-10000 - ll) = 0 in float64
        assert abs(-costs[0] - ll_bf) < 1e-10
        nll, g = tdt_autograd(x[0], labels[0], blank, durations, sigma)
        assert abs(nll - costs[0]) < 1e-10
        assert np.abs(g - grads[0]).max() < 1e-10
        assert abs(ex["ll_forward"][0] - ex["ll_backward"][0]) < 1e-10
        # rows of both logit-gradient blocks sum to zero
        assert np.abs(grads[0, :, :, :V].sum(-1)).max() < 1e-10
        assert np.abs(grads[0, :, :, V:].sum(-1)).max() < 1e-10


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("lam", [0.5, 0.01])
def test_fastemit_by_definition(impl, lam):
    """No reference vector covers TDT + FastEmit; this checks the kernel formula
    (gpu_rnnt_kernel.py:1363-1425) against its meaning: label-arc posteriors of
    the token branch scaled by (1+lambda), duration branch untouched."""
    rng = np.random.RandomState(19)
    durations = [0, 1, 2, 3]
    T, U, V = 6, 4, 5
    x = rng.randn(1, T, U, V + len(durations))
    labels = rng.randint(0, V - 1, size=(1, U - 1))
    costs, grads, _ = run_tdt(impl, x, labels, [T], [U - 1], V - 1, durations, 0.05, lam=lam)
    cost, g = tdt_autograd(x[0], labels[0], V - 1, durations, 0.05, lam=lam)
    assert abs(cost - costs[0]) < 1e-10
    assert np.abs(g - grads[0]).max() < 1e-10


@pytest.mark.parametrize("impl", IMPLS)
def test_closed_form_single_frame(impl):
    # T = 1: only duration-0 labels, then one duration-1 blank
    rng = np.random.RandomState(23)
    durations = [0, 1, 2]
    U, V, sigma = 4, 5, 0.07
    x = rng.randn(1, 1, U, V + 3)
    labels = rng.randint(0, V - 1, size=(1, U - 1))
    lp = log_softmax(x[0, 0, :, :V], axis=-1)
    dlp = log_softmax(x[0, 0, :, V:], axis=-1)
    ll = sum(lp[u, labels[0, u]] - sigma + dlp[u, 0] for u in range(U - 1)) + lp[U - 1, V - 1] - sigma + dlp[U - 1, 1]
    costs, _, _ = run_tdt(impl, x, labels, [1], [U - 1], V - 1, durations, sigma)
    assert abs(-costs[0] - ll) < 1e-12


@pytest.mark.parametrize("impl", IMPLS)
def test_closed_form_empty_transcript(impl):
    # U = 1: compositions of T into non-zero durations, a 1-D recursion over t
    rng = np.random.RandomState(29)
    durations = [0, 1, 2, 3]
    T, V, sigma = 7, 4, 0.05
    x = rng.randn(1, T, 1, V + 4)
    lp = log_softmax(x[0, :, 0, :V], axis=-1)
    dlp = log_softmax(x[0, :, 0, V:], axis=-1)
    f = np.full(T + 1, -np.inf)
    f[0] = 0.0
    for t in range(1, T + 1):
        f[t] = logsumexp(
            [f[t - d] + lp[t - d, V - 1] - sigma + dlp[t - d, i] for i, d in enumerate(durations) if d > 0 and t - d >= 0]
        )
    costs, _, _ = run_tdt(impl, x, np.zeros((1, 0), dtype=np.int64), [T], [0], V - 1, durations, sigma)
    assert abs(-costs[0] - f[T]) < 1e-12


@pytest.mark.parametrize("impl", IMPLS)
def test_variable_lengths_match_sliced_utterances(impl):
    rng = np.random.RandomState(31)
    durations = [0, 1, 2, 3, 4]
    B, T, U, V = 3, 9, 5, 6
    x = rng.randn(B, T, U, V + 5)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens = np.array([T, 4, 7])
    label_lens = np.array([2, U - 1, 0])
    costs, grads, _ = run_tdt(impl, x, labels, act_lens, label_lens, V - 1, durations, 0.05, lam=0.01, clamp=0.05)
    for b in range(B):
        tb, ub = act_lens[b], label_lens[b] + 1
        c1, g1, _ = run_tdt(
            impl, x[b : b + 1, :tb, :ub], labels[b : b + 1, : ub - 1], [tb], [ub - 1], V - 1, durations, 0.05,
            lam=0.01, clamp=0.05,
        )  # fmt: skip
        assert abs(c1[0] - costs[b]) < 1e-12
        assert np.abs(g1[0] - grads[b, :tb, :ub]).max() < 1e-12
        pad = grads[b].copy()
        pad[:tb, :ub] = 0
        assert np.all(pad == 0)


def test_c_matches_numpy_in_float64():
    rng = np.random.RandomState(37)
    B, T, U, V = 2, 8, 5, 7
    for durations in ([0, 1, 2, 3, 4], [1, 2, 4]):
        D = len(durations)
        x = rng.randn(B, T, U, V + D)
        labels = rng.randint(0, V - 1, size=(B, U - 1))
        act_lens = np.array([T, 5])
        label_lens = np.array([U - 1, 2])
        for lam, clamp in [(0.0, 0.0), (0.01, 0.0), (0.001, 0.02)]:
            c_n, g_n, e_n = onp.tdt_loss(x, labels, act_lens, label_lens, V - 1, durations, 0.05, lam, clamp)
            c_c, g_c, e_c = oracle.tdt_loss(x, labels, act_lens, label_lens, V - 1, durations, 0.05, lam, clamp)
            assert np.allclose(c_n, c_c, rtol=1e-13)
            assert np.abs(g_n - g_c).max() < 1e-13
            assert np.abs(e_n["duration_grads"] - e_c["duration_grads"]).max() < 1e-13


def test_durations_without_one_are_rejected():
    x = np.zeros((1, 3, 2, 6))
    with pytest.raises(RuntimeError):
        oracle.tdt_loss(x, [[0]], [3], [1], 3, [0, 2], 0.0)
    with pytest.raises(ValueError):
        onp.tdt_loss(x, [[0]], [3], [1], 3, [0, 2], 0.0)
