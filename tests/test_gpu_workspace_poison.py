"""Nothing the product leaves unwritten may reach a result.

Workspaces, gradient buffers and cost vectors are `torch.empty`: the kernels never write the lattice cells, arc
planes and coefficient records of padded cells, and readers are built so that whatever sits there cannot reach a
valid cell.  Here every `torch.empty` / `torch.empty_like` of the product modules is replaced by one that fills the
fresh tensor with a poison pattern (NaN, +Inf, -Inf as float64, all-ones bytes) and the costs and gradients of every
loss -- RNNT, TDT (both branches of omega), multi-blank, the compact log-prob op and the fused joint -- must come
out bit-identical to a run on zero-filled buffers, at ragged lengths, for float32 and bfloat16 logits.
"""

import numpy as np
import pytest
import torch

from gpu_utils import DEV, to_dev

pytestmark = pytest.mark.gpu


def _fill_fn(kind):
    def fill(t):
        if t.numel() == 0:
            return
        if kind == "zero":
            t.zero_()
        elif t.dtype == torch.uint8:
            if kind == "ff" or t.numel() % 8:
                t.fill_(255)
            elif kind == "nan":
                t.view(torch.float32).fill_(float("nan"))
            elif kind == "inf":
                t.view(torch.float32).fill_(float("inf"))
            else:  # "-inf64"
                t.view(torch.float64).fill_(float("-inf"))
        elif t.is_floating_point():
            t.fill_({"nan": float("nan"), "inf": float("inf"), "-inf64": float("-inf"), "ff": float("nan")}[kind])
        else:
            t.fill_(-1)

    return fill


class _PoisonTorch:
    """Stands in for the `torch` global of a product module: everything is forwarded, fresh tensors are poisoned."""

    def __init__(self, kind):
        self._fill = _fill_fn(kind)

    def __getattr__(self, name):
        return getattr(torch, name)

    def empty(self, *args, **kwargs):
        t = torch.empty(*args, **kwargs)
        self._fill(t)
        return t

    def empty_like(self, *args, **kwargs):
        t = torch.empty_like(*args, **kwargs)
        self._fill(t)
        return t


def _patched(monkeypatch, kind):
    import sys

    import speech_amd.joint.fused  # noqa: F401
    import speech_amd.k2  # noqa: F401
    from speech_amd.rnnt_loss import rnnt, rnnt_pytorch

    # (the package attribute of the same name is the function, hence the look-up by module name)
    k2, fused = sys.modules["speech_amd.k2.rnnt_logprobs"], sys.modules["speech_amd.joint.fused"]

    proxy = _PoisonTorch(kind)
    for mod in (rnnt, rnnt_pytorch, k2, fused):
        monkeypatch.setattr(mod, "torch", proxy)


def _inputs(seed, B, T, U, V, dtype):
    rng = np.random.RandomState(seed)
    x = torch.tensor(rng.randn(B, T, U, V) * 2.0, dtype=dtype)
    labels = rng.randint(0, V - 4, size=(B, U - 1))
    al = rng.randint(1, T + 1, size=B)
    ll = rng.randint(0, U, size=B)
    al[0], ll[-1] = T, U - 1
    al[-1], ll[0] = max(1, T // 3), 0  # a short utterance and one without labels
    return x, labels, al, ll


def _run_losses(dtype):
    """costs and gradients of every loss as a list of numpy arrays"""
    import random

    from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba
    from speech_amd.k2 import rnnt_logprobs

    out = []
    # three row-length classes of the two bandwidth passes: wave per row, workgroup per row, V small
    for V in (37, 300, 1030):
        B, T, U = 4, 11, 7
        x, labels, al, ll = _inputs(V, B, T, U, V, dtype)
        lab, ald, lld = to_dev(labels, al, ll)
        durations = [0, 1, 2, 3]
        cases = [
            RNNTLossNumba(blank=V - 1, reduction="none", fastemit_lambda=0.01, clamp=0.4),
            TDTLossNumba(blank=V - 5, durations=durations, reduction="none", sigma=0.05, omega=0.0),
            TDTLossNumba(blank=V - 5, durations=durations, reduction="none", sigma=0.05, omega=1.0),
            MultiblankRNNTLossNumba(blank=V - 1, big_blank_durations=[2, 4], reduction="none", sigma=0.05),
        ]
        for fn in cases:
            random.seed(0)
            acts = x.to(DEV).requires_grad_(True)
            costs = fn(acts, lab, ald, lld)
            costs.sum().backward()
            out += [costs.detach().float().cpu().numpy(), acts.grad.float().cpu().numpy()]
        logits = x.to(DEV).requires_grad_(True)
        ts, bs = rnnt_logprobs(logits, lab, V - 1, ald, lld)
        (ts.sum() + 2.0 * bs.sum()).backward()
        out += [ts.detach().cpu().numpy(), bs.detach().cpu().numpy(), logits.grad.float().cpu().numpy()]
    torch.cuda.synchronize()
    return out


def _run_joint():
    from speech_amd.joint import joint_multiblank_loss, joint_rnnt_loss, joint_tdt_loss

    rng = np.random.RandomState(5)
    B, T, U, V, H = 3, 21, 9, 133, 256  # utterances that end inside a 128-cell tile
    labels = rng.randint(0, V - 4, size=(B, U - 1))
    al, ll = np.array([T, 5, 13]), np.array([3, U - 1, 0])
    lab, ald, lld = to_dev(labels, al, ll)
    out = []
    for which in ("rnnt", "tdt", "multiblank"):
        f = torch.tensor(rng.randn(B, T, H), dtype=torch.bfloat16, device=DEV, requires_grad=True)
        g = torch.tensor(rng.randn(B, U, H), dtype=torch.bfloat16, device=DEV, requires_grad=True)
        rows = V + 3 if which == "tdt" else V
        w = torch.tensor(rng.randn(rows, H) / H**0.5, dtype=torch.float32, device=DEV, requires_grad=True)
        bias = torch.tensor(rng.randn(rows), dtype=torch.float32, device=DEV, requires_grad=True)
        if which == "rnnt":
            costs = joint_rnnt_loss(f, g, w, bias, lab, ald, lld, V - 1, 0.01, 0.3)
        elif which == "tdt":
            costs = joint_tdt_loss(f, g, w, bias, lab, ald, lld, V - 1, [0, 1, 2], 0.05)
        else:
            costs = joint_multiblank_loss(f, g, w, bias, lab, ald, lld, V - 1, [2, 3], 0.05)
        costs.sum().backward()
        out += [costs.detach().cpu().numpy()] + [p.grad.float().cpu().numpy() for p in (f, g, w, bias)]
    torch.cuda.synchronize()
    return out


def _assert_identical(got, want):
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.isfinite(b).all(), i
        assert np.array_equal(a, b), (i, float(np.nanmax(np.abs(a - b))))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_losses_ignore_what_fresh_buffers_hold(monkeypatch, dtype):
    _patched(monkeypatch, "zero")
    want = _run_losses(dtype)
    for kind in ("nan", "inf", "-inf64", "ff"):
        _patched(monkeypatch, kind)
        _assert_identical(_run_losses(dtype), want)


def test_fused_joint_ignores_what_fresh_buffers_hold(monkeypatch):
    _patched(monkeypatch, "zero")
    want = _run_joint()
    for kind in ("nan", "inf", "-inf64", "ff"):
        _patched(monkeypatch, kind)
        _assert_identical(_run_joint(), want)
