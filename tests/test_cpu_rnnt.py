"""The product's host (CPU) RNNT loss: speech_amd/csrc/mi_cpu.cpp behind RNNTLossNumba on CPU tensors and behind
rnnt_loss_cpu (rnnt.py:39-135).  Checked against the reference's golden vectors (its tests run every case on
DEVICES = ['cpu', ...], test_rnnt_pytorch.py:31-34) and against the oracle's restatement of the reference's CPU path
(oracle.rnnt_cpu_path: log_softmax, CPURNNT, softmax Jacobian, clamp hook).  Tolerances: the reference's own for the
golden vectors; 1e-5 relative on costs and 1e-5 absolute on gradients against the oracle (the reference keeps its
lattice in float32, the product in double, the oracle is run in double)."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import RNNTLossNumba, TDTLossNumba, MultiblankRNNTLossNumba
from speech_amd.rnnt_loss import rnnt


def call(fn, acts, labels, act_lens=None, label_lens=None, dtype=torch.float32):
    acts_t = torch.tensor(np.asarray(acts), dtype=dtype, requires_grad=True)
    B, T, U = acts_t.shape[:3]
    labels = torch.tensor(np.asarray(labels, dtype=np.int64).reshape(B, -1))
    al = torch.tensor(act_lens if act_lens is not None else [T] * B, dtype=torch.int64)
    ll = torch.tensor(label_lens if label_lens is not None else [labels.shape[1]] * B, dtype=torch.int64)
    costs = fn(acts_t, labels, al, ll)
    costs.sum().backward()
    return costs.detach().numpy(), acts_t.grad.float().numpy()


@pytest.mark.parametrize("name", ["small", "small_blank_last", "medium"])
def test_golden_vectors_on_cpu(golden, name):
    g = golden[name]
    costs, grads = call(RNNTLossNumba(blank=g["blank"], reduction='sum'), g["acts"], g["labels"])
    assert np.allclose(costs, sum(g["costs"]), atol=1e-8, rtol=1e-6)
    assert np.allclose(grads, np.array(g["grads"]), atol=1e-6, rtol=1e-3)


def test_golden_clamp_and_fastemit_cost_on_cpu(golden):
    g = golden["small_clamp"]
    costs, grads = call(RNNTLossNumba(blank=0, reduction='sum', clamp=g["clamp"]), g["acts"], g["labels"])
    assert np.allclose(costs, g["costs"], rtol=1e-6)
    assert np.allclose(grads, np.array(g["grads"]), atol=1e-7, rtol=1e-5)
    s = golden["small"]
    for lam in (1.0, 0.01, 0.00001):  # test_rnnt_pytorch.py:411-441
        costs, _ = call(RNNTLossNumba(blank=0, reduction='sum', fastemit_lambda=lam), s["acts"], s["labels"])
        assert np.allclose(costs, s["costs"][0] * (1.0 + lam), rtol=1e-6)


@pytest.mark.parametrize("seed,lam,clamp", [(0, 0.0, 0.0), (1, 0.01, 0.0), (2, 0.0, 0.05), (3, 0.001, 0.2)])
def test_ragged_batch_against_the_restated_reference_cpu_path(seed, lam, clamp):
    rng = np.random.RandomState(seed)
    B, T, U, V = 4, 9, 6, 11
    x = (rng.randn(B, T, U, V) * 2).astype(np.float32)
    labels = rng.randint(0, V, size=(B, U - 1))  # label == blank occurs
    al, ll = np.array([T, 3, 7, 1]), np.array([2, U - 1, 0, 4])
    blank = int(rng.randint(0, V))
    fn = RNNTLossNumba(blank=blank, reduction='none', fastemit_lambda=lam, clamp=clamp if clamp > 0 else -1)
    costs, grads = call(fn, x, labels, al, ll)
    c_ref, g_ref = oracle.rnnt_cpu_path(x, labels, al, ll, blank, lam, clamp, dtype=np.float64)
    np.testing.assert_allclose(costs, c_ref, rtol=1e-5)
    assert np.abs(grads - g_ref).max() < 1e-5
    for b in range(B):  # padded cells: exactly zero
        assert not grads[b, al[b]:].any() and not grads[b, :, ll[b] + 1:].any()


def test_reductions_grad_output_and_clamp_order():
    """'mean' divides costs and gradient by B (rnnt_pytorch.py:77-81), backward multiplies by grad_output (:88-92),
    and on the CPU the clamp hook sees the gradient after both (cpu_rnnt.py:141-161)."""
    rng = np.random.RandomState(5)
    B, T, U, V = 3, 5, 4, 6
    x = rng.randn(B, T, U, V).astype(np.float32)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    al, ll = [T, 4, 2], [U - 1, 1, 3]
    _, g_none = call(RNNTLossNumba(blank=V - 1, reduction='none'), x, labels, al, ll)
    c_sum, g_sum = call(RNNTLossNumba(blank=V - 1, reduction='sum'), x, labels, al, ll)
    c_mean, g_mean = call(RNNTLossNumba(blank=V - 1, reduction='mean'), x, labels, al, ll)
    assert c_sum.shape == (1,) and c_mean.shape == (1,)
    np.testing.assert_allclose(c_mean, c_sum / B, rtol=1e-6)
    np.testing.assert_allclose(g_sum, g_none, atol=1e-7)
    np.testing.assert_allclose(g_mean, g_none / B, atol=1e-7)
    # a per-utterance grad_output, then the clamp on the scaled gradient
    w = torch.tensor([2.0, -1.0, 0.5])
    acts = torch.tensor(x, requires_grad=True)
    fn = RNNTLossNumba(blank=V - 1, reduction='none', clamp=0.05)
    (fn(acts, torch.tensor(labels), torch.tensor(al), torch.tensor(ll)) * w).sum().backward()
    want = np.clip(g_none * w.numpy()[:, None, None, None], -0.05, 0.05)
    np.testing.assert_allclose(acts.grad.numpy(), want, atol=1e-7)


def test_sixteen_bit_cpu_logits_are_computed_in_float32():
    rng = np.random.RandomState(6)
    x = torch.tensor(rng.randn(2, 4, 3, 5), dtype=torch.float16)
    labels = rng.randint(0, 4, size=(2, 2))
    costs, grads = call(RNNTLossNumba(blank=4, reduction='none'), x.numpy(), labels, dtype=torch.float16)
    c_ref, g_ref = oracle.rnnt_cpu_path(x.float().numpy(), labels, [4, 4], [2, 2], 4, dtype=np.float64)
    assert costs.dtype == np.float32
    np.testing.assert_allclose(costs, c_ref, rtol=1e-5)
    assert np.abs(grads - g_ref).max() < 2.0**-10  # one float16 rounding of the gradient


def test_forward_only_and_errors():
    x = torch.zeros(1, 2, 2, 3)
    labels = torch.ones(1, 1, dtype=torch.int64)
    costs = RNNTLossNumba(blank=0, reduction='none')(x, labels, torch.tensor([2]), torch.tensor([1]))
    assert costs.shape == (1,) and not costs.requires_grad
    with pytest.raises(ValueError, match="Input length mismatch"):
        RNNTLossNumba()(x, labels, torch.tensor([1]), torch.tensor([1]))
    with pytest.raises(ValueError, match="clamp"):
        fn = RNNTLossNumba()
        fn.clamp = -1.0
        fn(x, labels, torch.tensor([2]), torch.tensor([1]))
    # the reference has no CPU path for these two either (rnnt_pytorch.py:137-140, :226-229)
    with pytest.raises(ValueError, match="non CUDA"):
        TDTLossNumba(blank=0, durations=[0, 1])(x, labels, torch.tensor([2]), torch.tensor([1]))
    with pytest.raises(NotImplementedError):
        MultiblankRNNTLossNumba(blank=2, big_blank_durations=[2])(x, labels, torch.tensor([2]), torch.tensor([1]))


def test_rnnt_loss_cpu_seam_leaves_the_sparse_log_prob_gradient():
    """rnnt_loss_cpu (rnnt.py:39-135) takes log-probs and fills the gradient w.r.t. them: two entries per cell.
    Taken through torch's log_softmax backward it must give the module's gradient."""
    rng = np.random.RandomState(7)
    B, T, U, V = 3, 6, 4, 7
    x = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32, requires_grad=True)
    labels = torch.tensor(rng.randint(0, V - 1, size=(B, U - 1)))
    al, ll = torch.tensor([T, 2, 5]), torch.tensor([1, U - 1, 0])
    log_probs = torch.log_softmax(x, -1)
    costs = torch.zeros(B)
    grads = torch.full_like(x, float('nan'))
    assert rnnt.rnnt_loss_cpu(log_probs.detach().contiguous(), labels, al, ll, costs, grads, V - 1, 0.01, 0.0, 2) is True
    assert (np.count_nonzero(grads.numpy(), axis=-1) <= 2).all()
    log_probs.backward(grads)
    c_mod, g_mod = call(RNNTLossNumba(blank=V - 1, reduction='none', fastemit_lambda=0.01), x.detach().numpy(),
                        labels.numpy(), al.tolist(), ll.tolist())
    np.testing.assert_allclose(costs.numpy(), c_mod, rtol=1e-6)
    np.testing.assert_allclose(x.grad.numpy(), g_mod, atol=1e-6)
    only = torch.zeros(B)
    assert rnnt.rnnt_loss_cpu(log_probs.detach().contiguous(), labels, al, ll, only, None, V - 1, 0.01, 0.0, -1) is True
    assert torch.equal(only, costs)
