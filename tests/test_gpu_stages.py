"""Entry points of the C ABI that the module path does not go through: the stage-by-stage calls (denominators,
lattice), the TDT function-level seam (tdt_loss_gpu, rnnt.py:239-363), the per-kernel timing hooks and the copy
probe of the benchmark."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import _native
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, to_dev

pytestmark = pytest.mark.gpu


def make(seed, B, T, U, V):
    rng = np.random.RandomState(seed)
    x = rng.randn(B, T, U, V).astype(np.float32)
    labels = rng.randint(0, 5, size=(B, U - 1))
    al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
    al[0], ll[-1] = T, U - 1
    return x, labels, al, ll


@pytest.mark.parametrize("with_betas", [False, True])
def test_denominators_then_lattice_is_the_forward_call(with_betas):
    B, T, U, V = 3, 13, 8, 70
    x, labels, al, ll = make(1, B, T, U, V)
    acts = torch.tensor(x, device=DEV)
    lab, ald, lld = to_dev(labels, al, ll)
    whole, split = (torch.empty(B, dtype=torch.float32, device=DEV) for _ in range(2))
    ws1, ws2 = rnnt.new_workspace(acts), rnnt.new_workspace(acts)
    rnnt.rnnt_forward(acts, lab, ald, lld, whole, V - 1, 0.01, with_betas, ws1)
    rnnt.denominators(acts, lab, ald, lld, V - 1, ws2)
    rnnt.rnnt_lattice(ald, lld, split, B, T, U, 0.01, with_betas, ws2)
    assert torch.equal(whole, split)
    c_ref, _, _ = oracle.rnnt_loss(x, labels, al, ll, V - 1, 0.01, 0.0)
    np.testing.assert_allclose(split.cpu().numpy(), c_ref, rtol=1e-6)
    # TDT: the same two stages with duration planes
    durations = [0, 1, 2]
    rnnt_x = np.random.RandomState(2).randn(B, T, U, V + 3).astype(np.float32)
    acts = torch.tensor(rnnt_x, device=DEV)
    ws1, ws2 = rnnt.new_workspace(acts, 3), rnnt.new_workspace(acts, 3)
    rnnt.tdt_forward(acts, lab, ald, lld, whole, V - 1, durations, 0.0, 0.05, False, with_betas, ws1)
    rnnt.denominators(acts, lab, ald, lld, V - 1, ws2, 3)
    rnnt.tdt_lattice(ald, lld, split, B, T, U, durations, 0.0, 0.05, with_betas, ws2)
    assert torch.equal(whole, split)
    c_ref, _, _ = oracle.tdt_loss(rnnt_x, labels, al, ll, V - 1, durations, 0.05)
    np.testing.assert_allclose(split.cpu().numpy(), c_ref, rtol=1e-6)


def test_combined_tdt_function_level_seam():
    B, T, U, V, durations = 3, 9, 5, 12, [0, 1, 2, 3]
    x, labels, al, ll = make(3, B, T, U, V + len(durations))
    acts = torch.tensor(x, device=DEV)
    lab, ald, lld = to_dev(labels, al, ll)
    costs = torch.zeros(B, device=DEV)
    grads = torch.full_like(acts, float('nan'))
    assert rnnt.combined_tdt_loss_gpu(acts, lab, ald, lld, costs, grads, V - 1, durations, 0.01, 0.2, 0, 0.05) is True
    c_ref, g_ref, _ = oracle.tdt_loss(x, labels, al, ll, V - 1, durations, 0.05, 0.01, 0.2)
    np.testing.assert_allclose(costs.cpu().numpy(), c_ref, rtol=1e-6)
    assert np.abs(grads.cpu().numpy() - g_ref).max() < 2e-6
    # grads None: forward only (rnnt.py:336-345)
    only = torch.zeros(B, device=DEV)
    assert rnnt.combined_tdt_loss_gpu(acts, lab, ald, lld, only, None, V - 1, durations, 0.01, 0.2, 0, 0.05) is True
    assert torch.equal(only, costs)
    with pytest.raises(TypeError):
        rnnt.combined_tdt_loss_gpu(acts, lab, ald, lld, costs.double(), None, V - 1, durations, 0.0, 0.0, 0, 0.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [12, 300, 1025])
def test_tdt_loss_gpu_with_the_reference_operands(dtype, V):
    """tdt_loss_gpu driven the way _TDTNumba.forward drives it (rnnt_pytorch.py:101-196): the caller splits the
    combined tensor, log-softmaxes the duration part and owns zero-filled costs / label_grads / duration_grads.
    label_grads is the gradient w.r.t. the token logits, duration_grads w.r.t. the duration LOG-PROBS
    (gpu_rnnt_kernel.py:1328-1341): both against the oracle's tdt_grads, which keeps them apart."""
    import random

    B, T, U, durations, sigma, lam, clamp = 3, 9, 5, [0, 1, 2, 3], 0.05, 0.01, 0.2
    D = len(durations)
    x, labels, al, ll = make(V, B, T, U, V + D)
    x = torch.tensor(x, dtype=dtype)
    lab, ald, lld = to_dev(labels, al, ll)
    label_acts = x[..., :V].contiguous().to(DEV)
    # the duration log-probs the kernels see are the caller's, rounded to the dtype of the logits
    duration_acts = torch.nn.functional.log_softmax(x[..., V:].float(), dim=-1).to(dtype).contiguous().to(DEV)
    # the oracle's per-utterance functions take log-probs for both parts, so they see exactly the (rounded,
    # hence not exactly normalised) duration log-probs that the kernels see
    from oracle import transducer_numpy as tn

    tok = x[..., :V].double().numpy()
    dlp = duration_acts.double().cpu().numpy()
    denom = tn.denominator(tok)
    c_ref = np.zeros(B)
    lg_ref, dg_ref = np.zeros((B, T, U, V)), np.zeros((B, T, U, D))
    for b in range(B):
        Tb, Ub = int(al[b]), int(ll[b]) + 1
        lp = tok[b] + denom[b][..., None]
        lab_b = [int(v) for v in labels[b][: Ub - 1]]
        a, llf = tn.tdt_alphas(lp, dlp[b], lab_b, Tb, Ub, V - 1, durations, sigma)
        bt, _ = tn.tdt_betas(lp, dlp[b], lab_b, Tb, Ub, V - 1, durations, sigma)
        lg, dg = tn.tdt_grads(lp, dlp[b], a, bt, llf, lab_b, Tb, Ub, V - 1, durations, sigma, lam, clamp)
        lg_ref[b, :Tb, :Ub], dg_ref[b, :Tb, :Ub] = lg, dg
        c_ref[b] = -llf * (1.0 + lam)
    f32 = dtype == torch.float32
    costs = torch.zeros(B, dtype=dtype, device=DEV)  # rnnt_pytorch.py:145: costs in the dtype of the logits
    label_grads = torch.full_like(label_acts, float('nan'))
    duration_grads = torch.full_like(duration_acts, float('nan'))
    assert rnnt.tdt_loss_gpu(label_acts, duration_acts, lab, ald, lld, costs, label_grads, duration_grads, V - 1,
                             durations, lam, clamp, 0, sigma, 0.0) is True  # fmt: skip
    np.testing.assert_allclose(costs.float().cpu().numpy(), c_ref, rtol=1e-5 if f32 else 2.0**-7)
    tol = 2e-6 if f32 else 2.0**-7
    assert np.abs(label_grads.float().cpu().numpy() - lg_ref).max() < tol
    assert np.abs(duration_grads.float().cpu().numpy() - dg_ref).max() < tol
    # duration_grads is minus an arc posterior: never positive, zero outside the utterance
    dg = duration_grads.float().cpu().numpy()
    assert (dg <= 0).all() and (dg[1, al[1]:] == 0).all()
    # forward only
    only = torch.zeros(B, dtype=torch.float32, device=DEV)
    assert rnnt.tdt_loss_gpu(label_acts, duration_acts, lab, ald, lld, only, None, None, V - 1, durations, lam,
                             clamp, 0, sigma, 0.0) is True  # fmt: skip
    np.testing.assert_allclose(only.cpu().numpy(), c_ref, rtol=1e-5 if f32 else 2.0**-7)
    # omega = 1: plain RNNT on the token logits, duration gradient zero (gpu_rnnt.py:606-682)
    random.seed(3)
    assert rnnt.tdt_loss_gpu(label_acts, duration_acts, lab, ald, lld, only, label_grads, duration_grads, V - 1,
                             durations, lam, clamp, 0, sigma, 1.0) is True  # fmt: skip
    c_r, g_r, _ = oracle.rnnt_loss(x[..., :V].float().numpy(), labels, al, ll, V - 1, lam, clamp)
    np.testing.assert_allclose(only.cpu().numpy(), c_r, rtol=1e-5)
    assert np.abs(label_grads.float().cpu().numpy() - g_r).max() < tol
    assert not duration_grads.any()
    with pytest.raises(ValueError):
        rnnt.tdt_loss_gpu(label_acts, duration_acts, lab, ald, lld, only, label_grads, None, V - 1, durations, lam,
                          clamp, 0, sigma, 0.0)  # fmt: skip


def test_timing_hooks_count_the_launches_they_bracket():
    B, T, U, V = 2, 7, 4, 33
    x, labels, al, ll = make(4, B, T, U, V)
    acts = torch.tensor(x, device=DEV)
    lab, ald, lld = to_dev(labels, al, ll)
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    grads = torch.empty_like(acts)
    ws = rnnt.new_workspace(acts)
    _native.profile_enable(8, ["denominator_pass", "lattice", "gradient_pass"])
    try:
        for _ in range(3):
            rnnt.rnnt_forward(acts, lab, ald, lld, costs, V - 1, 0.0, True, ws)
            rnnt.rnnt_backward(acts, lab, ald, lld, grads, None, V - 1, 0.0, 0.0, ws)
        torch.cuda.synchronize()
        got = _native.profile_read()
    finally:
        _native.profile_disable()
    for name in ("denominator_pass", "lattice", "gradient_pass"):
        ms, n = got[name]
        assert n == 3 and 0.0 < ms < 1000.0, (name, ms, n)
    assert got["zero_padding"][1] == 0
    # disabled again: nothing is recorded
    rnnt.rnnt_forward(acts, lab, ald, lld, costs, V - 1, 0.0, True, ws)
    torch.cuda.synchronize()
    assert all(n == 0 for _, n in _native.profile_read().values())


def test_copy_probe_copies():
    n = 1 << 20
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=DEV)
    dst = torch.zeros_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    assert _native.lib().mi_transducer_copy_probe(src.data_ptr(), dst.data_ptr(), n, stream) == _native.SUCCESS
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    assert _native.lib().mi_transducer_copy_probe(src.data_ptr(), dst.data_ptr(), n - 8, stream) == _native.INVALID_VALUE
    assert _native.lib().mi_transducer_copy_probe(src.data_ptr() + 4, dst.data_ptr(), n - 16, stream) == _native.INVALID_VALUE


def test_work_is_enqueued_on_the_current_stream():
    """The reference picks torch's current stream (rnnt.py:173-176).  Here: inputs produced on a side stream, the
    loss called there without any synchronisation in between, the result consumed there -- right only if every
    kernel of forward and backward went to that stream (a slow kernel ahead of the producer makes a miss show)."""
    from speech_amd import RNNTLossNumba

    B, T, U, V = 4, 40, 12, 257
    x, labels, al, ll = make(5, B, T, U, V)
    lab, ald, lld = to_dev(labels, al, ll)
    base = torch.tensor(x, device=DEV)
    ref_acts = (base * 2 + 1).requires_grad_(True)
    ref = RNNTLossNumba(blank=V - 1, reduction='none')(ref_acts, lab, ald, lld)
    ref.sum().backward()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    big = torch.randn(4096, 4096, device=DEV)
    with torch.cuda.stream(side):
        for _ in range(20):
            big = big @ big * 1e-3  # keeps the side stream busy ahead of the producer below
        acts = (base * 2 + 1).requires_grad_(True)
        costs = RNNTLossNumba(blank=V - 1, reduction='none')(acts, lab, ald, lld)
        costs.sum().backward()
        got_c, got_g = costs.detach().clone(), acts.grad.clone()
    side.synchronize()
    assert torch.equal(got_c, ref.detach()) and torch.equal(got_g, ref_acts.grad)
