"""Logits and gradients whose storage does not start on a 16-byte boundary.

`acts = big[1:]...` is a contiguous tensor whose base is element-aligned only.  Two things are checked against the
oracle, for RNNT, TDT (both omega branches) and the multi-blank loss, float32 and bfloat16, over vocabulary sizes of
every row-length class:
  * through the module surface the gradient buffer is allocated at the logits' phase, so the vector kernels run;
  * through the function-level seam with a caller-owned gradient buffer at ANOTHER phase the library takes its
    element-wise kernels (cell coefficients + scalar stores), which must give the same numbers.
Tolerances: north-star bar (costs 1e-5 relative, gradients 1e-4 absolute) for float32; one bfloat16 rounding step
(2^-8 relative to the largest entry) for bfloat16 gradients.
"""

import random

import numpy as np
import pytest
import torch

import oracle
from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, to_dev

pytestmark = pytest.mark.gpu

DURATIONS = [0, 1, 2]
BIG_BLANKS = [2, 3]


def shifted(x, shift):
    """A contiguous device copy of x whose first element sits `shift` elements past a 16-byte boundary."""
    flat = torch.empty(x.numel() + 16, dtype=x.dtype, device=DEV)
    assert flat.data_ptr() % 16 == 0
    view = flat[shift : shift + x.numel()].view(x.shape)
    view.copy_(x)
    assert (view.data_ptr() & 15) == (shift * x.element_size()) % 16
    return view


def case(seed, V, extra, dtype):
    rng = np.random.RandomState(seed)
    B, T, U = 3, 9, 6
    x = torch.tensor(rng.randn(B, T, U, V + extra) * 2.0, dtype=dtype)
    labels = rng.randint(0, V - 3, size=(B, U - 1))
    al, ll = np.array([T, 4, 7]), np.array([2, U - 1, 0])
    return x, labels, al, ll


def reference(kind, x, labels, al, ll, V):
    xf = x.float().numpy()
    if kind == "rnnt":
        return oracle.rnnt_loss(xf, labels, al, ll, V - 1, 0.01, 0.3)[:2]
    if kind == "tdt":
        return oracle.tdt_loss(xf, labels, al, ll, V - 1, DURATIONS, 0.05, 0.01, 0.3)[:2]
    if kind == "tdt_omega":  # plain RNNT on the token logits, zero gradient for the duration logits
        c, g, _ = oracle.rnnt_loss(xf[..., :V], labels, al, ll, V - 1, 0.01, 0.3)
        return c, np.concatenate([g, np.zeros(g.shape[:3] + (len(DURATIONS),), g.dtype)], axis=-1)
    return oracle.multiblank_loss(xf, labels, al, ll, V - 1, BIG_BLANKS, 0.05, 0.01, 0.3)[:2]


def module_of(kind, V):
    if kind == "rnnt":
        return RNNTLossNumba(blank=V - 1, reduction="none", fastemit_lambda=0.01, clamp=0.3)
    if kind in ("tdt", "tdt_omega"):
        return TDTLossNumba(blank=V - 1, durations=DURATIONS, reduction="none", fastemit_lambda=0.01, clamp=0.3,
                            sigma=0.05, omega=1.0 if kind == "tdt_omega" else 0.0)  # fmt: skip
    return MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=BIG_BLANKS, reduction="none",
                                   fastemit_lambda=0.01, clamp=0.3, sigma=0.05)  # fmt: skip


def check(costs, grads, c_ref, g_ref, dtype, costs_dtype=torch.float32):
    # the costs are computed in float32 from the logits as given; TDT and multi-blank modules then round them to
    # the dtype of the logits (rnnt_pytorch.py:145, :232)
    np.testing.assert_allclose(costs, c_ref, rtol=1e-5 if costs_dtype == torch.float32 else 2.0**-7)
    if dtype == torch.float32:
        assert np.abs(grads - g_ref).max() < 1e-4
    else:
        assert np.abs(grads - g_ref).max() <= 2.0**-8 * max(1.0, np.abs(g_ref).max())


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "tdt_omega", "multiblank"])
@pytest.mark.parametrize("dtype,shift", [(torch.float32, 1), (torch.float32, 3), (torch.bfloat16, 1), (torch.bfloat16, 6)])
@pytest.mark.parametrize("V", [5, 37, 259, 1025, 2051])
def test_module_on_a_shifted_view(kind, dtype, shift, V):
    extra = len(DURATIONS) if kind.startswith("tdt") else 0
    x, labels, al, ll = case(V + shift, V, extra, dtype)
    acts = shifted(x, shift).requires_grad_(True)
    lab, ald, lld = to_dev(labels, al, ll)
    random.seed(1)
    costs = module_of(kind, V)(acts, lab, ald, lld)
    costs.sum().backward()
    assert acts.grad.shape == acts.shape
    c_ref, g_ref = reference(kind, x, labels, al, ll, V)
    check(costs.detach().float().cpu().numpy(), acts.grad.float().cpu().numpy(), c_ref, g_ref, dtype, costs.dtype)


@pytest.mark.parametrize("kind", ["rnnt", "tdt", "tdt_omega", "multiblank"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [5, 259, 1025])
def test_function_seam_with_gradients_at_another_phase(kind, dtype, V):
    extra = len(DURATIONS) if kind.startswith("tdt") else 0
    x, labels, al, ll = case(V, V, extra, dtype)
    acts = shifted(x, 1)
    lab, ald, lld = to_dev(labels, al, ll)
    costs = torch.zeros(x.shape[0], dtype=torch.float32, device=DEV)
    c_ref, g_ref = reference(kind, x, labels, al, ll, V)
    for grad_shift in (0, 2):  # neither is the phase of acts
        grads = shifted(torch.full(x.shape, float("nan"), dtype=dtype), grad_shift)
        if kind == "rnnt":
            rnnt.rnnt_loss_gpu(acts, lab, ald, lld, costs, grads, V - 1, 0.01, 0.3, 0)
        elif kind == "multiblank":
            rnnt.multiblank_rnnt_loss_gpu(acts, lab, ald, lld, costs, grads, V - 1, BIG_BLANKS, 0.01, 0.3, 0, 0.05)
        else:
            rnnt.combined_tdt_loss_gpu(acts, lab, ald, lld, costs, grads, V - 1, DURATIONS, 0.01, 0.3, 0, 0.05,
                                       kind == "tdt_omega")  # fmt: skip
        torch.cuda.synchronize()
        check(costs.cpu().numpy(), grads.float().cpu().numpy(), c_ref, g_ref, dtype)
