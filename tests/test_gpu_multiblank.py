"""GPU parity of the multi-blank transducer loss (through the C ABI) against the oracle."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, multiblank_rnnt_loss_gpu
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, call_loss, make_lengths, to_dev
from helpers import multiblank_autograd

pytestmark = pytest.mark.gpu


def check_against_oracle(acts, labels, act_lens, label_lens, blank, durs, sigma, lam=0.0, clamp=0.0, reduction='none',
                         cost_rtol=1e-6, grad_atol=2e-6, dtype=torch.float32):  # fmt: skip
    fn = MultiblankRNNTLossNumba(blank=blank, big_blank_durations=durs, reduction=reduction, fastemit_lambda=lam,
                                 clamp=clamp if clamp > 0 else -1, sigma=sigma)  # fmt: skip
    costs, grads = call_loss(fn, acts, labels, act_lens, label_lens, dtype=dtype)
    x = torch.as_tensor(np.asarray(acts), dtype=dtype).float().numpy()
    c_ref, g_ref, _ = oracle.multiblank_loss(x, labels, act_lens, label_lens, blank, durs, sigma, lam, clamp, num_threads=4)
    if reduction == 'sum':
        c_ref = c_ref.sum(keepdims=True)
    assert costs.shape == c_ref.shape
    assert np.allclose(costs, c_ref, rtol=cost_rtol, atol=0), (costs, c_ref)
    err = np.abs(grads - g_ref).max()
    assert err < grad_atol, err
    return costs, grads


def test_reference_randomized_case_against_autograd():
    """Shapes of the reference's only multi-blank test (test_rnnt_pytorch.py:510-541): B,T,U,V = 4,8,4,8,
    durations [2,4,8], sigma 0.1, reduction 'sum'; there the numba kernels are compared with torch autograd
    of a pure-Python recursion (rtol 1e-2 on gradients), here with autograd of an alpha-only recursion."""
    rng = np.random.RandomState(0)
    B, T, U, V = 4, 8, 4, 8
    durs, sigma = [2, 4, 8], 0.1
    acts = rng.rand(B, T, U, V + 1 + len(durs))
    labels = rng.randint(0, V, size=(B, U - 1))
    blank = V + len(durs)
    fn = MultiblankRNNTLossNumba(blank=blank, reduction='sum', big_blank_durations=durs, sigma=sigma)
    cost, grads = call_loss(fn, acts, labels)
    ag = [multiblank_autograd(acts[b], labels[b], blank, durs, sigma) for b in range(B)]
    assert np.allclose(cost, sum(a[0] for a in ag), rtol=1e-6)
    assert np.abs(grads - np.stack([a[1] for a in ag])).max() < 2e-6


@pytest.mark.parametrize("durs", [[], [2], [2, 4], [2, 4, 8], [3, 5, 7, 9, 11], [2, 3, 4, 5, 6, 7, 8, 9]])
def test_variable_lengths_fastemit_clamp(durs):
    rng = np.random.RandomState(len(durs) + 40)
    B, T, U, Vtok = 4, 17, 7, 11
    V = Vtok + len(durs) + 1
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, Vtok, size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, 2, 0)
    costs, grads = check_against_oracle(acts, labels, act_lens, label_lens, V - 1, durs, 0.05, lam=0.01, clamp=0.2)
    for b in range(B):
        pad = grads[b].copy()
        pad[: act_lens[b], : label_lens[b] + 1] = 0
        assert np.all(pad == 0)


@pytest.mark.parametrize("V", [29, 301, 1028, 5003])
def test_row_lengths_of_every_kernel_family(V):
    rng = np.random.RandomState(V)
    durs = [2, 4, 8]
    B, T, U = 2, 9, 4
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1 - len(durs), size=(B, U - 1))
    check_against_oracle(acts, labels, np.array([T, 5]), np.array([1, U - 1]), V - 1, durs, 0.05, lam=0.001)


@pytest.mark.parametrize("U", [1, 2, 65, 130])
def test_label_axis_sizes(U):
    rng = np.random.RandomState(U)
    durs = [2, 4]
    B, T, V = 2, 12, 9
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 3, size=(B, U - 1))
    check_against_oracle(acts, labels, np.array([T, 5]), np.array([U - 1, (U - 1) // 2]), V - 1, durs, 0.1)


@pytest.mark.parametrize("U,durs", [(300, [2, 3, 4, 5, 6, 7, 8, 9]), (513, [2, 4, 8]), (1024, [2, 4]), (1024, [2, 3, 4, 5, 6, 7, 8, 9])])
def test_label_axes_whose_ring_exceeds_lds(U, durs):
    """When (longest big blank + 1) x (2 + big blanks) x U doubles pass 160 KB the lattice is computed by the
    kernel that pulls alphas / betas from global memory; its values are those of the LDS-ring kernel."""
    rng = np.random.RandomState(U + len(durs))
    B, T = 2, 23
    V = 7 + len(durs)
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1 - len(durs), size=(B, U - 1))
    # hundreds of log-sum-exp steps of up to ten terms: float rounding of the gradients reaches 5e-6 (the bar is 1e-4)
    check_against_oracle(acts, labels, np.array([T, 14]), np.array([U - 1, (U - 1) // 2]), V - 1, durs, 0.05, grad_atol=1e-5)


@pytest.mark.parametrize(
    "shape,durs,lens",
    [
        ((1, 15, 11, 6), [2, 3, 4], None),          # utils/test_gpu_rnnt_kernel.py:711-797 (alphas) and :800-886 (betas)
        ((3, 40, 17, 12), [2, 4, 8], "ragged"),     # ragged lengths, a blank longer than some utterances' remainders
        ((2, 23, 300, 15), [2, 3, 4, 5, 6, 7, 8, 9], "ragged"),  # the ring exceeds LDS: the kernel that pulls from memory
    ],
)
def test_stage_level_lattice(shape, durs, lens):
    """The forward variables, the backward variables and both log-likelihoods on their own, read out of the workspace
    after the forward call (the reference tests its multi-blank alpha and beta kernels on their own too): an error
    in alpha or beta that cancels in the gradient would not show in the end-to-end tests."""
    B, T, U, V = shape
    rng = np.random.RandomState(U + len(durs))
    x = rng.randn(B, T, U, V).astype(np.float32)
    labels = rng.randint(0, V - 1 - len(durs), size=(B, U - 1))
    if lens is None:
        act_lens, label_lens = [T] * B, [U - 1] * B
    else:
        act_lens, label_lens = make_lengths(rng, B, T, U, 3, 0)
    acts = torch.tensor(x, device=DEV)
    lab, al, ll = to_dev(labels, act_lens, label_lens)
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    ws = rnnt.new_workspace(acts, len(durs))
    rnnt.multiblank_forward(acts, lab, al, ll, costs, V - 1, durs, 0.0, 0.05, True, ws)
    denom, alphas, betas, llf, llb = [t.cpu().numpy() for t in rnnt.export_lattice(ws, al, ll, B, T, U, len(durs))]
    c_ref, _, ex = oracle.multiblank_loss(x, labels, act_lens, label_lens, V - 1, durs, 0.05, want_grads=False)
    valid = (np.arange(T)[None, :, None] < np.asarray(act_lens)[:, None, None]) & (
        np.arange(U)[None, None, :] <= np.asarray(label_lens)[:, None, None]
    )
    assert np.abs(denom - ex["denom"])[valid].max() < 1e-5
    # (cells no alignment reaches hold -inf in the oracle and the kernels' large negative stand-in here: compare
    # the reachable ones, and require the others to be far below any reachable value)
    for got, want in ((alphas, ex["alphas"]), (betas, ex["betas"])):
        reach = valid & np.isfinite(want)
        assert reach.any() and np.abs(got - want)[reach].max() < 2e-4 * max(1.0, np.abs(want[reach]).max() / 50)
        assert np.all(got[valid & ~np.isfinite(want)] < want[reach].min() - 100)
    assert np.allclose(llf, ex["ll_forward"], rtol=1e-6, atol=1e-5) and np.allclose(llb, llf, rtol=1e-6, atol=1e-5)
    assert np.allclose(costs.cpu().numpy(), c_ref, rtol=1e-6)


def test_blank_in_the_middle_and_reductions_and_half_precision():
    rng = np.random.RandomState(77)
    B, T, U, V = 3, 10, 5, 12
    durs, blank = [2, 3], 6  # big blanks at 5 and 4
    acts = rng.randn(B, T, U, V)
    labels = rng.choice([0, 1, 2, 3, 7, 8, 9, 10, 11], size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, 3, 1)
    check_against_oracle(acts, labels, act_lens, label_lens, blank, durs, 0.05, reduction='sum')
    # 16-bit logits: the costs come back in the dtype of acts (rnnt_pytorch.py:232), i.e. rounded to bf16
    check_against_oracle(acts, labels, act_lens, label_lens, blank, durs, 0.05, lam=0.01, cost_rtol=2.0**-8,
                         grad_atol=2.0**-8, dtype=torch.bfloat16)  # fmt: skip


def test_without_big_blanks_and_sigma_it_is_the_rnnt_loss():
    rng = np.random.RandomState(5)
    B, T, U, V = 2, 9, 4, 7
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    c_mb, g_mb = call_loss(MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=[], reduction='none'), acts, labels)
    c_r, g_r = call_loss(RNNTLossNumba(blank=V - 1, reduction='none'), acts, labels)
    assert np.allclose(c_mb, c_r, rtol=1e-6) and np.abs(g_mb - g_r).max() < 2e-6


def test_function_level_seam_and_errors():
    rng = np.random.RandomState(9)
    B, T, U, V, durs = 2, 6, 3, 8, [2, 4]
    acts = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32, device=DEV)
    labels = rng.randint(0, V - 3, size=(B, U - 1))
    lab, al, ll = to_dev(labels, [T] * B, [U - 1] * B)
    costs = torch.zeros(B, device=DEV)
    grads = torch.zeros_like(acts)
    assert multiblank_rnnt_loss_gpu(acts, lab, al, ll, costs, grads, V - 1, durs, 0.0, 0.0, 0, 0.05) is True
    c_ref, g_ref, _ = oracle.multiblank_loss(acts.cpu().numpy(), labels, [T] * B, [U - 1] * B, V - 1, durs, 0.05)
    assert np.allclose(costs.cpu().numpy(), c_ref, rtol=1e-6)
    assert np.abs(grads.cpu().numpy() - g_ref).max() < 2e-6
    with pytest.raises(NotImplementedError):  # no CPU path, as in the reference (rnnt_pytorch.py:226-229)
        MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=durs)(acts.cpu(), lab.cpu(), al.cpu(), ll.cpu())
    with pytest.raises(RuntimeError):  # a duration beyond the supported range
        MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=[2, 100])(acts, lab, al, ll)
