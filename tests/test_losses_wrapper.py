"""The model-facing wrapper (speech_amd.losses.rnnt) against the behaviour of
nemo/collections/asr/losses/rnnt.py:88-505.  CPU part: resolution, validation, errors.  GPU part
(marked): reductions, casting, padded inputs, all three loss names."""

import logging

import numpy as np
import pytest
import torch

from speech_amd.losses import RNNT_LOSS_RESOLVER, RNNTLoss, resolve_rnnt_default_loss_name, resolve_rnnt_loss
from speech_amd.rnnt_loss import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba


def test_resolver_table_has_the_reference_names():
    # losses/rnnt.py:88-158
    assert set(RNNT_LOSS_RESOLVER) == {
        "warprnnt", "warprnnt_numba", "pytorch", "multiblank_rnnt", "multiblank_rnnt_pytorch", "graph_w_transducer",
        "graph_rnnt", "tdt", "tdt_pytorch", "default",
    }  # fmt: skip
    assert RNNT_LOSS_RESOLVER["default"] is RNNT_LOSS_RESOLVER["warprnnt_numba"]
    assert resolve_rnnt_default_loss_name() == "warprnnt_numba"
    assert [n for n, c in RNNT_LOSS_RESOLVER.items() if c.is_available] == ["warprnnt_numba", "multiblank_rnnt", "tdt", "default"]


def test_resolution_and_kwargs(caplog):
    loss = resolve_rnnt_loss("default", blank_idx=28, loss_kwargs={"fastemit_lambda": 0.01, "clamp": 2.0})
    assert isinstance(loss, RNNTLossNumba)
    assert (loss.blank, loss.reduction, loss.fastemit_lambda, loss.clamp) == (28, 'none', 0.01, 2.0)
    loss = resolve_rnnt_loss("warprnnt_numba", blank_idx=5)
    assert (loss.fastemit_lambda, loss.clamp) == (0.0, 0.0)  # clamp=-1.0 is stored as 0.0 (rnnt_pytorch.py:409)
    loss = resolve_rnnt_loss("tdt", 1024, {"durations": [0, 1, 2, 3, 4], "sigma": 0.05, "omega": 0.1})
    assert isinstance(loss, TDTLossNumba) and loss.durations == [0, 1, 2, 3, 4] and loss.sigma == 0.05 and loss.omega == 0.1
    loss = resolve_rnnt_loss("multiblank_rnnt", 1027, {"big_blank_durations": [2, 4, 8], "sigma": 0.05})
    assert isinstance(loss, MultiblankRNNTLossNumba) and loss.big_blank_durations == [2, 4, 8] and loss.blank == 1027
    kwargs = {"fastemit_lambda": 0.0, "not_an_argument": 3}
    with caplog.at_level(logging.WARNING):
        resolve_rnnt_loss("warprnnt_numba", 5, kwargs)
    assert "not_an_argument" in caplog.text and "ignored" in caplog.text
    assert kwargs == {"fastemit_lambda": 0.0, "not_an_argument": 3}  # the caller's dict is left alone


def test_errors():
    with pytest.raises(ValueError, match="not in list of available RNNT losses"):
        resolve_rnnt_loss("ctc", 5)
    for name in ["warprnnt", "pytorch", "graph_rnnt", "graph_w_transducer", "tdt_pytorch", "multiblank_rnnt_pytorch"]:
        with pytest.raises(ImportError, match="Installed RNNT losses are"):
            resolve_rnnt_loss(name, 5)
    with pytest.raises(ValueError, match="`reduction` must be one of"):
        RNNTLoss(num_classes=5, reduction="average")
    loss = RNNTLoss(num_classes=5)
    assert loss.reduction == "mean_batch" and loss._blank == 5 and loss._loss.reduction == 'none'
    x = torch.zeros(1, 2, 2, 6)
    with pytest.raises(TypeError, match="passed by kwargs only"):
        loss(x, torch.zeros(1, 1), torch.tensor([2]), torch.tensor([1]))


def test_reduce_matches_the_reference_formulas():
    # losses/rnnt.py:421-436
    losses, tl = torch.tensor([2.0, 6.0, 9.0]), torch.tensor([1, 2, 3])
    expect = {None: None, "sum": 17.0, "mean_batch": 17.0 / 3, "mean": (2.0 + 3.0 + 3.0) / 3, "mean_volume": 17.0 / 6}
    for red, val in expect.items():
        if red is None:
            continue
        assert abs(float(RNNTLoss(4, reduction=red).reduce(losses, tl)) - val) < 1e-6
    # lists of per-sub-batch results are concatenated first (the fused joint/loss step does that)
    out = RNNTLoss(4, reduction="mean_volume").reduce([losses[:1], losses[1:]], [tl[:1], tl[1:]])
    assert abs(float(out) - 17.0 / 6) < 1e-6


# ------------------------------------------------------------------------------------- GPU

gpu = pytest.mark.gpu


def _case(rng, B, T, U, V, t_lo, u_lo):
    from gpu_utils import make_lengths

    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, t_lo, u_lo)
    return acts, labels, act_lens, label_lens


@gpu
@pytest.mark.parametrize("reduction", [None, "sum", "mean_batch", "mean", "mean_volume"])
def test_rnnt_reductions_and_int32_inputs(reduction):
    import oracle
    from gpu_utils import DEV

    rng = np.random.RandomState(3)
    B, T, U, V = 4, 11, 6, 9
    acts, labels, act_lens, label_lens = _case(rng, B, T, U, V, 3, 1)
    x = torch.tensor(acts, dtype=torch.float32, device=DEV, requires_grad=True)
    loss = RNNTLoss(num_classes=V - 1, reduction=reduction, loss_kwargs={"fastemit_lambda": 0.01})
    out = loss(
        log_probs=x,
        targets=torch.tensor(labels, dtype=torch.int32, device=DEV),  # cast to int64 by the wrapper (:441-443)
        input_lengths=torch.tensor(act_lens, dtype=torch.int32, device=DEV),
        target_lengths=torch.tensor(label_lens, dtype=torch.int32, device=DEV),
    )
    c, g, _ = oracle.rnnt_loss(acts.astype(np.float32), labels, act_lens, label_lens, V - 1, 0.01, 0.0)
    tl = label_lens.astype(np.float64)
    w = {None: np.ones(B), "sum": np.ones(B), "mean_batch": np.full(B, 1 / B), "mean": 1 / tl / B,
         "mean_volume": np.full(B, 1 / tl.sum())}[reduction]  # fmt: skip
    expect = c if reduction is None else (c * w).sum()
    assert out.dtype == torch.float32 and out.shape == ((B,) if reduction is None else ())
    assert np.allclose(out.detach().cpu().numpy(), expect, rtol=1e-6)
    out.sum().backward()
    assert np.abs(x.grad.cpu().numpy() - g * w[:, None, None, None]).max() < 2e-6
    assert loss._loss.reduction == 'none'  # restored after the call (:484-491)


@gpu
def test_time_axis_longer_than_the_lengths_and_wide_target_matrix():
    """The reference narrows both (:473-481); here the full tensors go in and the result is the same, with a
    zero gradient on the extra frames."""
    import oracle
    from gpu_utils import DEV

    rng = np.random.RandomState(4)
    B, T, U, V, extra = 3, 9, 5, 8, 4
    acts, labels, act_lens, label_lens = _case(rng, B, T, U, V, 3, 1)
    padded = np.concatenate([acts, rng.randn(B, extra, U, V)], axis=1)
    wide = np.concatenate([labels, rng.randint(0, V - 1, size=(B, 3))], axis=1)
    x = torch.tensor(padded, dtype=torch.float32, device=DEV, requires_grad=True)
    loss = RNNTLoss(num_classes=V - 1, reduction="sum")
    out = loss(log_probs=x, targets=torch.tensor(wide, device=DEV), input_lengths=torch.tensor(act_lens, device=DEV),
               target_lengths=torch.tensor(label_lens, device=DEV))  # fmt: skip
    c, g, _ = oracle.rnnt_loss(acts.astype(np.float32), labels, act_lens, label_lens, V - 1)
    assert np.allclose(float(out.detach()), c.sum(), rtol=1e-6)
    out.backward()
    grad = x.grad.cpu().numpy()
    assert np.abs(grad[:, :T] - g).max() < 2e-6 and np.all(grad[:, T:] == 0)
    # a length beyond the tensor is still an error
    with pytest.raises(ValueError, match="Input length mismatch"):
        loss(log_probs=x, targets=torch.tensor(wide, device=DEV),
             input_lengths=torch.tensor([T + extra + 1] * B, device=DEV),
             target_lengths=torch.tensor(label_lens, device=DEV))  # fmt: skip
    # and the module on its own keeps the reference's exact check (rnnt_pytorch.py:628-634)
    with pytest.raises(ValueError, match="Input length mismatch"):
        RNNTLossNumba(blank=V - 1)(x, torch.tensor(labels, device=DEV), torch.tensor(act_lens, device=DEV),
                                   torch.tensor(label_lens, device=DEV))  # fmt: skip


@gpu
def test_tdt_and_multiblank_by_name_and_16_bit_joint():
    import oracle
    from gpu_utils import DEV

    rng = np.random.RandomState(6)
    B, T, U, Vtok = 3, 10, 5, 9
    # TDT: blank id = num_classes = V, duration logits after it
    durs = [0, 1, 2]
    acts, labels, act_lens, label_lens = _case(rng, B, T, U, Vtok + 1 + len(durs), 3, 1)
    labels = labels % Vtok
    x = torch.tensor(acts, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    loss = RNNTLoss(num_classes=Vtok, reduction=None, loss_name="tdt", loss_kwargs={"durations": durs, "sigma": 0.05})
    out = loss(log_probs=x, targets=torch.tensor(labels, device=DEV), input_lengths=torch.tensor(act_lens, device=DEV),
               target_lengths=torch.tensor(label_lens, device=DEV))  # fmt: skip
    xf = x.detach().float().cpu().numpy()
    c, g, _ = oracle.tdt_loss(xf, labels, act_lens, label_lens, Vtok, durs, 0.05)
    assert out.dtype == torch.float32  # the reference's wrapper computes 16-bit joints in fp32 (:449-465)
    assert np.allclose(out.detach().cpu().numpy(), c, rtol=1e-6)
    out.sum().backward()
    assert x.grad.dtype == torch.bfloat16 and np.abs(x.grad.float().cpu().numpy() - g).max() < 2.0**-8
    # multi-blank: blank id = num_classes = V + number of big blanks
    big = [2, 4]
    acts, labels, act_lens, label_lens = _case(rng, B, T, U, Vtok + len(big) + 1, 3, 1)
    labels = labels % Vtok
    x = torch.tensor(acts, dtype=torch.float16, device=DEV, requires_grad=True)
    loss = RNNTLoss(num_classes=Vtok + len(big), reduction="mean_batch", loss_name="multiblank_rnnt",
                    loss_kwargs={"big_blank_durations": big, "sigma": 0.05})  # fmt: skip
    out = loss(log_probs=x, targets=torch.tensor(labels, device=DEV), input_lengths=torch.tensor(act_lens, device=DEV),
               target_lengths=torch.tensor(label_lens, device=DEV))  # fmt: skip
    c, g, _ = oracle.multiblank_loss(x.detach().float().cpu().numpy(), labels, act_lens, label_lens, Vtok + len(big), big, 0.05)
    assert out.dtype == torch.float32 and np.allclose(float(out.detach()), c.mean(), rtol=1e-6)
    out.backward()
    assert np.abs(x.grad.float().cpu().numpy() - g / B).max() < 2.0**-11
