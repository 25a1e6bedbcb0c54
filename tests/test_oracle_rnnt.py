"""Pins the RNNT oracle (numpy loops and the C restatement, f32 and f64)
against the reference's golden vectors and against independent mathematics."""

import numpy as np
import pytest
from scipy.special import logsumexp

import oracle
from oracle import transducer_numpy as onp

from helpers import rnnt_autograd, rnnt_bruteforce_ll, rnnt_fastemit_autograd

IMPLS = ["numpy", "c"]


def run_rnnt(impl, acts, labels, act_lens, label_lens, blank, lam=0.0, clamp=0.0, dtype=np.float64):
    if impl == "numpy":
        return onp.rnnt_loss(acts, labels, act_lens, label_lens, blank, lam, clamp, dtype=dtype)
    return oracle.rnnt_loss(acts, labels, act_lens, label_lens, blank, lam, clamp, dtype=dtype)


def test_lse_known_answer(golden):
    # tests/collections/asr/numba/rnnt_loss/utils/test_rnnt_helper.py:42-61
    k = golden["lse_kat"]
    total = sum(onp.lse2(np.float64(k["a"]), np.float64(k["b"])) for _ in range(k["times"]))
    assert abs(total - k["expected_sum"]) < 1e-12
    assert onp.lse2(-np.inf, 3.0) == 3.0 and onp.lse2(3.0, -np.inf) == 3.0
    assert onp.lse2(-np.inf, -np.inf) == -np.inf


def test_denominator_closed_form():
    rng = np.random.RandomState(1)
    x = rng.randn(3, 4, 5, 17) * 3
    assert np.allclose(onp.denominator(x), -logsumexp(x, axis=-1), atol=1e-13)


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name", ["small", "small_blank_last", "medium"])
def test_golden_vectors(golden, impl, name):
    g = golden[name]
    costs, grads, ex = run_rnnt(impl, g["acts"], g["labels"], g["act_lens"], g["label_lens"], g["blank"])
    # small / medium literals carry 7-8 correct digits; small_blank_last was
    # produced in float32 (its literals are float32 values printed in full)
    atol = 1e-6 if name == "small_blank_last" else 2e-8
    assert np.allclose(costs, g["costs"], rtol=2e-7, atol=0)
    assert np.allclose(grads, np.array(g["grads"]), atol=atol, rtol=1e-5)
    assert np.allclose(ex["ll_forward"], ex["ll_backward"], atol=1e-12)


@pytest.mark.parametrize("impl", IMPLS)
def test_golden_vectors_float32(golden, impl):
    # the reference's own tolerance for fp32: cost atol 1e-8/rtol 1e-6, grads rtol 1e-5..1e-3
    for name in ["small", "small_blank_last", "medium"]:
        g = golden[name]
        costs, grads, _ = run_rnnt(
            impl, g["acts"], g["labels"], g["act_lens"], g["label_lens"], g["blank"], dtype=np.float32
        )
        assert costs.dtype == np.float32
        assert np.allclose(costs, g["costs"], rtol=1e-6)
        assert np.allclose(grads, np.array(g["grads"]), atol=1e-6, rtol=1e-3)


@pytest.mark.parametrize("impl", IMPLS)
def test_golden_clamp(golden, impl):
    g = golden["small_clamp"]
    costs, grads, _ = run_rnnt(
        impl, g["acts"], g["labels"], g["act_lens"], g["label_lens"], g["blank"], clamp=g["clamp"]
    )
    assert np.allclose(costs, g["costs"], rtol=2e-7)
    assert np.allclose(grads, np.array(g["grads"]), atol=2e-8, rtol=1e-5)


@pytest.mark.parametrize("impl", IMPLS)
def test_golden_fastemit_cost(golden, impl):
    g = golden["small"]
    for lam in golden["fastemit_lambdas"]:
        costs, grads, _ = run_rnnt(impl, g["acts"], g["labels"], g["act_lens"], g["label_lens"], g["blank"], lam=lam)
        assert np.allclose(costs, g["costs"][0] * (1.0 + lam), rtol=2e-7)
        # every row of a logits-gradient sums to zero (softmax Jacobian)
        assert np.abs(grads.sum(-1)).max() < 1e-12


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("blank_pos", ["first", "last", "middle"])
def test_bruteforce_and_autograd(impl, blank_pos):
    rng = np.random.RandomState(7)
    for T, U, V in [(1, 1, 3), (1, 4, 4), (4, 1, 3), (3, 3, 4), (5, 4, 5), (2, 5, 6)]:
        blank = {"first": 0, "last": V - 1, "middle": V // 2}[blank_pos]
        x = rng.randn(1, T, U, V) * 2
        choices = [v for v in range(V) if v != blank]
        labels = rng.choice(choices, size=(1, max(U - 1, 0)))
        costs, grads, ex = run_rnnt(impl, x, labels, [T], [U - 1], blank)
        ll = rnnt_bruteforce_ll(x[0], labels[0], blank)
        assert abs(-costs[0] - ll) < 1e-11
        nll, g = rnnt_autograd(x[0], labels[0], blank)
        assert abs(nll - costs[0]) < 1e-11
        assert np.abs(g - grads[0]).max() < 1e-11
        assert abs(ex["ll_forward"][0] - ex["ll_backward"][0]) < 1e-11


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("lam", [1.0, 0.01, 0.001])
def test_fastemit_gradient_by_definition(impl, lam):
    rng = np.random.RandomState(11)
    T, U, V, blank = 5, 4, 6, 5
    x = rng.randn(1, T, U, V)
    labels = rng.randint(0, V - 1, size=(1, U - 1))
    costs, grads, _ = run_rnnt(impl, x, labels, [T], [U - 1], blank, lam=lam)
    cost, g = rnnt_fastemit_autograd(x[0], labels[0], blank, lam)
    assert abs(cost - costs[0]) < 1e-11
    assert np.abs(g - grads[0]).max() < 1e-11


@pytest.mark.parametrize("impl", IMPLS)
def test_label_equal_to_blank_id(impl):
    # pathological but legal for the kernels: both sparse terms hit the same logit
    rng = np.random.RandomState(3)
    T, U, V, blank = 4, 3, 4, 1
    x = rng.randn(1, T, U, V)
    labels = np.array([[1, 2]])
    costs, grads, _ = run_rnnt(impl, x, labels, [T], [U - 1], blank, lam=0.5)
    cost, g = rnnt_fastemit_autograd(x[0], labels[0], blank, 0.5)
    assert abs(cost - costs[0]) < 1e-11
    assert np.abs(g - grads[0]).max() < 1e-11


@pytest.mark.parametrize("impl", IMPLS)
def test_variable_lengths_match_sliced_utterances(impl):
    # tests/collections/asr/conftest.py:324-347 shape of the variable-length generator
    rng = np.random.RandomState(2021)
    B, T, U, V, blank = 4, 12, 9, 8, 7
    x = rng.rand(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens = np.array([T, T // 2, U - 1, 3])
    label_lens = np.array([U - 1, U - 2, U - 4, 0])
    costs, grads, ex = run_rnnt(impl, x, labels, act_lens, label_lens, blank, lam=0.01, clamp=0.05)
    for b in range(B):
        tb, ub = act_lens[b], label_lens[b] + 1
        c1, g1, _ = run_rnnt(
            impl, x[b : b + 1, :tb, :ub], labels[b : b + 1, : ub - 1], [tb], [ub - 1], blank, lam=0.01, clamp=0.05
        )
        assert abs(c1[0] - costs[b]) < 1e-12
        assert np.abs(g1[0] - grads[b, :tb, :ub]).max() < 1e-12
        pad = grads[b].copy()
        pad[:tb, :ub] = 0
        assert np.all(pad == 0)


def test_c_matches_numpy_exactly_in_float64():
    rng = np.random.RandomState(5)
    B, T, U, V, blank = 3, 9, 7, 11, 10
    x = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens = np.array([T, 5, 7])
    label_lens = np.array([3, U - 1, 0])
    for lam, clamp in [(0.0, 0.0), (0.01, 0.0), (0.001, 0.02)]:
        c_n, g_n, e_n = onp.rnnt_loss(x, labels, act_lens, label_lens, blank, lam, clamp)
        c_c, g_c, e_c = oracle.rnnt_loss(x, labels, act_lens, label_lens, blank, lam, clamp)
        assert np.allclose(c_n, c_c, rtol=1e-14)
        assert np.abs(g_n - g_c).max() < 1e-14
        for b in range(B):
            tb, ub = act_lens[b], label_lens[b] + 1
            assert np.allclose(e_n["alphas"][b, :tb, :ub], e_c["alphas"][b, :tb, :ub], atol=1e-12)
            assert np.allclose(e_n["betas"][b, :tb, :ub], e_c["betas"][b, :tb, :ub], atol=1e-12)
            assert np.allclose(e_n["denom"][b, :tb, :ub], e_c["denom"][b, :tb, :ub], atol=1e-13)


def test_posterior_invariants():
    # for every t < T-1 the blank arcs leaving row t carry total posterior 1,
    # and so do the label arcs leaving column u for every u < U-1
    rng = np.random.RandomState(9)
    T, U, V, blank = 7, 5, 6, 0
    x = rng.randn(1, T, U, V)
    labels = rng.randint(1, V, size=(1, U - 1))
    _, _, ex = oracle.rnnt_loss(x, labels, [T], [U - 1], blank)
    lp = x[0] + ex["denom"][0][..., None]
    a, b, ll = ex["alphas"][0], ex["betas"][0], ex["ll_forward"][0]
    for t in range(T - 1):
        assert abs(logsumexp(a[t, :] + lp[t, :, blank] + b[t + 1, :]) - ll) < 1e-11
    for u in range(U - 1):
        assert abs(logsumexp(a[:, u] + lp[:, u, labels[0, u]] + b[:, u + 1]) - ll) < 1e-11


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_cpu_path_matches_gpu_semantics(dtype):
    """The reference's CPU path (sparse log-prob gradient + softmax Jacobian + clamp
    hook) and its GPU path (dense logits-gradient) are the same function."""
    rng = np.random.RandomState(13)
    B, T, U, V, blank = 3, 10, 6, 9, 8
    x = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens = np.array([T, 6, 9])
    label_lens = np.array([U - 1, 2, 4])
    tol = 1e-12 if dtype == np.float64 else 2e-6
    for lam, clamp in [(0.0, 0.0), (0.01, 0.0), (0.0, 0.03)]:
        c_g, g_g, _ = oracle.rnnt_loss(x, labels, act_lens, label_lens, blank, lam, clamp, dtype=dtype)
        c_c, g_c = oracle.rnnt_cpu_path(x, labels, act_lens, label_lens, blank, lam, clamp, dtype=dtype, num_threads=2)
        assert np.allclose(c_g, c_c, rtol=tol * 10)
        assert np.abs(g_g - g_c).max() < tol


def test_invalid_lengths_are_rejected():
    x = np.zeros((1, 3, 2, 4))
    with pytest.raises(RuntimeError):
        oracle.rnnt_loss(x, [[1]], [4], [1], 0)
    with pytest.raises(RuntimeError):
        oracle.rnnt_loss(x, [[1]], [3], [2], 0)
