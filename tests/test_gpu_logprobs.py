"""GPU parity of the compact log-prob op (mi_rnnt_logprobs_forward / _backward through speech_amd.k2)
against the oracle.  Tolerances: 1e-5 absolute on scores and gradients for float32 (what the reference's
own test allows, tests/collections/asr/k2/test_graph_transducer.py:326-336); 16-bit logits are compared
with the oracle on the upcast logits, the gradient within one rounding step of the 16-bit type."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd.k2 import rnnt_logprobs, rnnt_logprobs_triton

from gpu_utils import DEV

pytestmark = pytest.mark.gpu


def run_case(rng, B, T, U, V, blank, dtype=torch.float32, ragged=False, scale=1.0, keep=True, int32_lengths=False,
             score_atol=1e-5, grad_atol=1e-5):  # fmt: skip
    logits_np = (rng.rand(B, T, U, V) * scale).astype(np.float32)
    lo = 1 if blank == 0 else 0
    targets = rng.randint(lo, V - 1 + lo, size=(B, U - 1))
    src = tgt = None
    if ragged:
        src = rng.randint(1, T + 1, size=B)
        tgt = rng.randint(0, U, size=B)
    logits = torch.tensor(logits_np, dtype=dtype, device=DEV, requires_grad=True)
    x = logits.detach().float().cpu().numpy()
    len_dtype = torch.int32 if int32_lengths else torch.int64
    kw = {}
    if ragged:
        kw = dict(source_lengths=torch.tensor(src, dtype=len_dtype, device=DEV),
                  target_lengths=torch.tensor(tgt, dtype=len_dtype, device=DEV))  # fmt: skip
    ts, bs = rnnt_logprobs(logits, torch.tensor(targets, device=DEV), blank, keep_forward_state=keep, **kw)
    assert ts.dtype == torch.float32 and ts.shape == (B, T, U) and bs.shape == (B, T, U)
    ts_ref, bs_ref = oracle.rnnt_logprobs(x, targets, blank, src, tgt)
    assert np.abs(ts.detach().cpu().numpy() - ts_ref).max() < score_atol
    assert np.abs(bs.detach().cpu().numpy() - bs_ref).max() < score_atol
    gt = rng.rand(B, T, U).astype(np.float32)
    gb = rng.rand(B, T, U).astype(np.float32)
    (torch.tensor(gt, device=DEV) * ts + torch.tensor(gb, device=DEV) * bs).sum().backward()
    torch.cuda.synchronize()
    g_ref = oracle.rnnt_logprobs_grad(x, targets, blank, gt, gb, src, tgt)
    g = logits.grad
    assert g.dtype == dtype and g.shape == logits.shape
    err = np.abs(g.float().cpu().numpy() - g_ref).max()
    assert err < grad_atol, err
    return ts, bs, g


@pytest.mark.parametrize("shape", [(1, 4, 2, 4), (2, 3, 2, 5), (2, 16, 31, 17), (16, 129, 65, 2048)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_reference_shapes(shape, dtype):
    """The four shapes of test_rnnt_logprobs_random (test_graph_transducer.py:281-336): uniform [0,1)
    logits [B, T, U+1, V+1], blank id = V, full lengths, random upstream gradients."""
    B, T, Utext, Vtok = shape
    rng = np.random.RandomState(777)
    # a bf16 gradient entry near 1 is rounded to 2^-8 relative
    run_case(rng, B, T, Utext + 1, Vtok + 1, Vtok, dtype=dtype, grad_atol=1e-5 if dtype == torch.float32 else 2.0**-8)


@pytest.mark.parametrize("V", [2, 3, 64, 129, 1025, 4099, 20000])
@pytest.mark.parametrize("blank_first", [False, True])
def test_ragged_lengths_every_row_length(V, blank_first):
    rng = np.random.RandomState(V)
    ts, bs, g = run_case(rng, 3, 9, 6, V, 0 if blank_first else V - 1, ragged=True, scale=4.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sixteen_bit_logits_ragged(dtype):
    rng = np.random.RandomState(11)
    run_case(rng, 4, 12, 7, 515, 514, dtype=dtype, ragged=True, scale=3.0, grad_atol=2.0**-8)


def test_backward_without_forward_state_and_int32_lengths():
    rng = np.random.RandomState(12)
    run_case(rng, 3, 10, 5, 300, 299, ragged=True, keep=False, int32_lengths=True)


def test_padding_is_exactly_zero_and_independent_of_its_logits():
    rng = np.random.RandomState(13)
    B, T, U, V = 3, 8, 5, 40
    x = rng.randn(B, T, U, V).astype(np.float32)
    targets = rng.randint(0, V - 1, size=(B, U - 1))
    src, tgt = np.array([8, 3, 5]), np.array([2, 4, 0])
    outs = []
    for fill in (0.0, np.nan):
        y = x.copy()
        for b in range(B):
            y[b, src[b] :] = fill
            y[b, :, tgt[b] + 1 :] = fill
        logits = torch.tensor(y, device=DEV, requires_grad=True)
        ts, bs = rnnt_logprobs_triton(logits, torch.tensor(targets, device=DEV), V - 1,
                                      torch.tensor(src, device=DEV), torch.tensor(tgt, device=DEV))  # fmt: skip
        (ts.sum() + 2 * bs.sum()).backward()
        outs.append((ts.detach().cpu().numpy(), bs.detach().cpu().numpy(), logits.grad.cpu().numpy()))
    for a, b_ in zip(outs[0], outs[1]):
        assert np.array_equal(a, b_)
    ts, bs, g = outs[0]
    for b in range(B):
        assert np.all(ts[b, src[b] :] == 0) and np.all(ts[b, :, tgt[b] :] == 0)
        assert np.all(bs[b, src[b] :] == 0) and np.all(bs[b, :, tgt[b] + 1 :] == 0)
        assert np.all(g[b, src[b] :] == 0) and np.all(g[b, :, tgt[b] + 1 :] == 0)


def test_target_equal_to_blank_follows_the_reference_kernel():
    rng = np.random.RandomState(14)
    B, T, U, V = 2, 3, 4, 6
    x = rng.randn(B, T, U, V).astype(np.float32)
    targets = np.array([[5, 1, 5], [0, 5, 2]])
    logits = torch.tensor(x, device=DEV, requires_grad=True)
    ts, bs = rnnt_logprobs(logits, torch.tensor(targets, device=DEV), 5)
    gt, gb = rng.rand(2, B, T, U).astype(np.float32)
    (torch.tensor(gt, device=DEV) * ts + torch.tensor(gb, device=DEV) * bs).sum().backward()
    g_ref = oracle.rnnt_logprobs_grad(x, targets, 5, gt, gb)
    assert np.abs(logits.grad.cpu().numpy() - g_ref).max() < 1e-6


def test_input_checks():
    logits = torch.zeros(2, 3, 4, 5, device=DEV)
    with pytest.raises(ValueError):
        rnnt_logprobs(logits, torch.zeros(2, 4, dtype=torch.int64, device=DEV), 4)
    with pytest.raises(RuntimeError):
        rnnt_logprobs(logits.cpu(), torch.zeros(2, 3, dtype=torch.int64), 4)
    with pytest.raises(RuntimeError):  # blank id outside the vocabulary: invalid value from the library
        rnnt_logprobs(logits, torch.zeros(2, 3, dtype=torch.int64, device=DEV), 5)
