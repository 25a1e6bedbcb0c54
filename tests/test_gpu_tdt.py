"""GPU parity of the TDT loss against the oracle and the reference's fixed vector."""

import random

import numpy as np
import pytest
import torch

import oracle
from speech_amd import TDTLossNumba
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, call_loss, make_lengths, to_dev

pytestmark = pytest.mark.gpu


def check_against_oracle(acts, labels, act_lens, label_lens, blank, durations, sigma, lam=0.0, clamp=0.0,
                         cost_rtol=1e-6, grad_atol=2e-6, dtype=torch.float32):  # fmt: skip
    fn = TDTLossNumba(blank=blank, durations=durations, reduction='none', fastemit_lambda=lam,
                      clamp=clamp if clamp > 0 else -1, sigma=sigma)  # fmt: skip
    costs, grads = call_loss(fn, acts, labels, act_lens, label_lens, dtype=dtype)
    x = torch.as_tensor(np.asarray(acts), dtype=dtype).float().numpy()
    c_ref, g_ref, _ = oracle.tdt_loss(x, labels, act_lens, label_lens, blank, durations, sigma, lam, clamp, num_threads=4)
    assert np.allclose(costs, c_ref, rtol=cost_rtol, atol=0), (costs, c_ref)
    err = np.abs(grads - g_ref).max()
    assert err < grad_atol, err
    return costs, grads


def test_golden_fixed_vector(golden):
    g = golden["tdt_fixed"]
    fn = TDTLossNumba(blank=g["blank"], reduction='sum', durations=g["durations"], sigma=g["sigma"])
    costs, grads = call_loss(fn, np.zeros(g["shape"]), g["labels"])
    assert np.allclose(costs, g["costs"], rtol=1e-6)
    assert np.allclose(grads, np.array(g["grads"]), atol=1e-6, rtol=1e-4)


@pytest.mark.parametrize("durations", [[0, 1, 2, 3, 4, 5], [1, 2, 3, 4, 5], [0, 1], [1], [0, 1, 2, 3, 4]])
def test_random_cases_like_the_reference(durations):
    # test_rnnt_pytorch.py:547-589: B,T,U,V = 4,8,4,8, uniform logits, sigma 0.05, with and without duration 0
    rng = np.random.RandomState(len(durations) * 10 + durations[0])
    B, T, U, V = 4, 8, 4, 8
    acts = rng.rand(B, T, U, V + 1 + len(durations))
    labels = rng.randint(0, V, size=(B, U - 1))
    check_against_oracle(acts, labels, [T] * B, [U - 1] * B, V, durations, 0.05)


@pytest.mark.parametrize("V", [4, 29, 301, 1025, 2500, 5001])
def test_variable_lengths_fastemit_clamp(V):
    rng = np.random.RandomState(V + 1)
    durations = [0, 1, 2, 3, 4]
    B, T, U = 4, 14, 8
    acts = rng.randn(B, T, U, V + 5)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, 2, 0)
    costs, grads = check_against_oracle(acts, labels, act_lens, label_lens, V - 1, durations, 0.05, lam=0.01, clamp=0.2)
    for b in range(B):
        pad = grads[b].copy()
        pad[: act_lens[b], : label_lens[b] + 1] = 0
        assert np.all(pad == 0)


@pytest.mark.parametrize("U", [1, 65, 130])
def test_label_axis_sizes(U):
    rng = np.random.RandomState(U)
    durations = [0, 1, 2, 4]
    B, T, V = 2, 9, 6
    acts = rng.randn(B, T, U, V + 4)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    check_against_oracle(acts, labels, [T, 5], [U - 1, (U - 1) // 3], V - 1, durations, 0.02)


@pytest.mark.parametrize("U,durations", [(300, [0, 1, 2, 3, 4]), (513, [0, 1, 2, 3, 4, 5, 6, 7, 8]), (1024, [0, 1, 2, 4, 8])])
def test_label_axes_beyond_the_paired_lattice_kernel(U, durations):
    """More than 256 label columns run the one-wave-per-direction lattice kernel, whose ring of arc scores
    grows with U and the longest duration (up to the whole LDS of a CU at U = 1024, durations to 8)."""
    rng = np.random.RandomState(U)
    B, T, V = 2, 17, 6
    acts = rng.randn(B, T, U, V + len(durations))
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    # 500+ log-sum-exp steps of up to nine terms each: float rounding of the gradients reaches 2e-6 (the bar is 1e-4)
    check_against_oracle(acts, labels, [T, 11], [U - 1, (U - 1) // 3], V - 1, durations, 0.02, grad_atol=1e-5)


def test_stage_level_lattice():
    # shape of utils/test_gpu_rnnt_kernel.py:617-708: [1,15,11,3] token + [1,15,11,3] duration logits
    rng = np.random.RandomState(0)
    durations = [0, 1, 2]
    B, T, U, V = 1, 15, 11, 3
    x = rng.randn(B, T, U, V + 3)
    labels = rng.randint(1, V, size=(B, U - 1))
    acts = torch.tensor(x, dtype=torch.float32, device=DEV)
    lab, al, ll = to_dev(labels, [T], [U - 1])
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    ws = rnnt.new_workspace(acts, 3)
    rnnt.tdt_forward(acts, lab, al, ll, costs, 0, durations, 0.0, 0.05, False, True, ws)
    denom, alphas, betas, llf, llb = [t.cpu().numpy() for t in rnnt.export_lattice(ws, al, ll, B, T, U, 3)]
    _, _, ex = oracle.tdt_loss(x.astype(np.float32), labels, [T], [U - 1], 0, durations, 0.05)
    assert np.abs(denom - ex["denom"]).max() < 1e-6
    assert np.abs(alphas - ex["alphas"]).max() < 1e-5
    assert np.abs(betas - ex["betas"]).max() < 1e-5
    assert abs(llf[0] - ex["ll_forward"][0]) < 1e-5 and abs(llb[0] - llf[0]) < 1e-5


def test_omega_one_is_the_plain_rnnt_loss_on_the_token_logits():
    rng = np.random.RandomState(21)
    durations = [0, 1, 2, 3]
    B, T, U, V = 3, 10, 5, 11
    acts = rng.randn(B, T, U, V + 4)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, 2, 0)
    random.seed(0)
    fn = TDTLossNumba(blank=V - 1, durations=durations, reduction='none', sigma=0.05, omega=1.0, fastemit_lambda=0.01)
    costs, grads = call_loss(fn, acts, labels, act_lens, label_lens)
    x = acts.astype(np.float32)
    c_ref, g_ref, _ = oracle.rnnt_loss(x[..., :V], labels, act_lens, label_lens, V - 1, 0.01)
    assert np.allclose(costs, c_ref, rtol=1e-6)
    assert np.abs(grads[..., :V] - g_ref).max() < 2e-6
    assert np.all(grads[..., V:] == 0)


def test_costs_follow_the_dtype_of_acts_and_cpu_raises_value_error():
    durations = [0, 1, 2]
    acts = torch.randn(1, 4, 3, 8, device=DEV, dtype=torch.bfloat16)
    lab, al, ll = to_dev([[1, 2]], [4], [2])
    fn = TDTLossNumba(blank=4, durations=durations, reduction='none', sigma=0.05)
    assert fn(acts, lab, al, ll).dtype == torch.bfloat16
    with pytest.raises(ValueError, match="non CUDA"):
        fn(acts.cpu().float(), lab.cpu(), al.cpu(), ll.cpu())
    with pytest.raises(RuntimeError):
        TDTLossNumba(blank=4, durations=[0, 2, 3], reduction='none')(acts, lab, al, ll)  # no duration 1


@pytest.mark.parametrize("durations", [[1, 2], [1, 3], [1, 2, 4], [0, 1, 2]])
def test_utterances_without_an_alignment_follow_the_sentinel_arithmetic(durations):
    """Without a duration 0 every label needs a frame of its own: more labels than frames leave no alignment, and the
    reference's result is what its -10000 sentinels add up to (cost about 10000 plus a few arc log-probs).  The
    forward log-likelihood then shows how the final sum is formed -- the duration-1 term is assigned, not added to
    the -10000 it starts from (gpu_rnnt_kernel.py:1046-1071) -- so these costs pin that detail.  With duration 0 in
    the set the same shapes are ordinary cases."""
    rng = np.random.RandomState(len(durations) * 7 + durations[-1])
    B, T, U, V = 4, 6, 9, 12
    D = len(durations)
    acts = rng.randn(B, T, U, V + D)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens = np.array([6, 2, 3, 1])
    label_lens = np.array([8, 5, 3, 4])
    fn = TDTLossNumba(blank=V - 1, durations=durations, reduction='none', sigma=0.05)
    costs, grads = call_loss(fn, acts, labels, act_lens, label_lens)
    c_ref, g_ref, _ = oracle.tdt_loss(acts.astype(np.float32), labels, act_lens, label_lens, V - 1, durations, 0.05)
    if durations[0] != 0:
        assert np.all(c_ref > 9000)
    np.testing.assert_allclose(costs, c_ref, rtol=2e-6)
    assert np.abs(grads - g_ref).max() <= 1e-5 * max(1.0, np.abs(g_ref).max())
