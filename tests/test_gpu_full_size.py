"""The five benchmark configurations at their full sizes.

The oracle is too slow for a multi-GB tensor, so each configuration is checked
(1) against the oracle on whole utterances cut out of the batch (the loss is
independent per utterance), and (2) through properties that hold at any size:
padded cells exactly zero, every valid gradient row sums to zero (no clamp),
forward and backward likelihoods agree, the gradient is linear in grad_output,
and two runs are bit-identical.
Bar (north star): costs within 1e-5 relative, gradients within 1e-4 absolute
(fp32); for bf16 the gradient is additionally rounded to bf16 on store.
"""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import RNNTLossNumba, TDTLossNumba, synthetic
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV

pytestmark = pytest.mark.gpu

COST_RTOL = 1e-5
GRAD_ATOL = 1e-4


def make_loss(cfg, reduction='none'):
    if cfg.D:
        return TDTLossNumba(blank=cfg.blank, durations=cfg.durations, reduction=reduction,
                            fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp, sigma=cfg.sigma)  # fmt: skip
    return RNNTLossNumba(blank=cfg.blank, reduction=reduction, fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp)


def oracle_utterance(cfg, acts, labels, act_lens, label_lens, b):
    tb, ub = int(act_lens[b]), int(label_lens[b]) + 1
    x = acts[b : b + 1, :tb, :ub].float().cpu().numpy()
    lab = labels[b : b + 1, : ub - 1].cpu().numpy()
    lam, clamp = cfg.fastemit_lambda, max(cfg.clamp, 0.0)
    if cfg.D:
        c, g, _ = oracle.tdt_loss(x, lab, [tb], [ub - 1], cfg.blank, cfg.durations, cfg.sigma, lam, clamp, num_threads=1)
    else:
        c, g, _ = oracle.rnnt_loss(x, lab, [tb], [ub - 1], cfg.blank, lam, clamp, num_threads=1)
    return c[0], g[0]


@pytest.mark.parametrize("index", [1, 2, 3, 4])
def test_full_size_configuration(index):
    cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(index, device=DEV, generate_on_device=True)
    acts.requires_grad_(True)
    loss = make_loss(cfg)
    costs = loss(acts, labels, act_lens, label_lens)
    costs.sum().backward()
    grads = acts.grad
    torch.cuda.synchronize()
    assert costs.shape == (cfg.B,) and bool(torch.isfinite(costs).all()) and bool((costs > 0).all())

    # (1) whole utterances against the float64 oracle: the two smallest lattices
    cells = (act_lens * (label_lens + 1)).cpu().numpy()
    grad_eps = GRAD_ATOL if cfg.dtype == torch.float32 else GRAD_ATOL + 2.0**-8
    for b in np.argsort(cells)[:2]:
        b = int(b)
        tb, ub = int(act_lens[b]), int(label_lens[b]) + 1
        c_ref, g_ref = oracle_utterance(cfg, acts.detach(), labels, act_lens, label_lens, b)
        cb = float(costs[b].detach())
        assert abs(cb - c_ref) <= COST_RTOL * abs(c_ref), (b, cb, c_ref)
        got = grads[b, :tb, :ub].float().cpu().numpy()
        err = np.abs(got - g_ref).max()
        assert err < grad_eps, (b, err)

    # (2a) padded cells are exactly zero
    T, U = cfg.T, cfg.U
    t_idx = torch.arange(T, device=DEV).view(1, T, 1)
    u_idx = torch.arange(U, device=DEV).view(1, 1, U)
    valid = (t_idx < act_lens.view(-1, 1, 1)) & (u_idx <= label_lens.view(-1, 1, 1))
    for b in range(cfg.B):
        pad_abs = grads[b].float().abs().amax(dim=-1)[~valid[b]]
        assert pad_abs.numel() == 0 or float(pad_abs.max()) == 0.0
    # (2b) without a clamp every valid row of the logits-gradient sums to zero (token and duration blocks apart)
    if cfg.clamp <= 0:
        V = cfg.V
        tol = 2e-5 if cfg.dtype == torch.float32 else 0.1  # bf16 rounding of ~1000 stored entries
        for b in range(cfg.B):
            g = grads[b].float()
            assert float(g[..., :V].sum(-1).abs().max()) < tol
            if cfg.D:
                assert float(g[..., V:].sum(-1).abs().max()) < tol
    del grads

    # (2c) forward and backward likelihoods agree
    ws = rnnt.new_workspace(acts, cfg.D)
    c2 = torch.empty(cfg.B, dtype=torch.float32, device=DEV)
    if cfg.D:
        rnnt.tdt_forward(acts.detach(), labels, act_lens, label_lens, c2, cfg.blank, cfg.durations,
                         cfg.fastemit_lambda, cfg.sigma, False, True, ws)  # fmt: skip
    else:
        rnnt.rnnt_forward(acts.detach(), labels, act_lens, label_lens, c2, cfg.blank, cfg.fastemit_lambda, True, ws)
    _, _, _, llf, llb = rnnt.export_lattice(ws, act_lens, label_lens, cfg.B, cfg.T, cfg.U, cfg.D)
    assert float(((llf - llb).abs() / llf.abs()).max()) < 1e-6
    assert torch.equal(c2.to(costs.dtype), costs.detach())  # (2e) bit-identical second run
    del ws

    # (2d) linear in grad_output, and (2e) deterministic
    first = acts.grad.clone()
    acts.grad = None
    w = torch.linspace(0.5, 2.0, cfg.B, device=DEV)
    (loss(acts, labels, act_lens, label_lens).float() * w).sum().backward()
    probe = [0, cfg.B // 2, cfg.B - 1]
    for b in probe:
        want = first[b].float() * float(w[b])
        tol = 1e-6 if cfg.dtype == torch.float32 else 2.0**-7 * float(want.abs().max())
        assert float((acts.grad[b].float() - want).abs().max()) <= tol
    acts.grad = None
    loss(acts, labels, act_lens, label_lens).sum().backward()
    assert torch.equal(acts.grad, first)


def test_full_size_configuration_1_against_the_whole_oracle():
    cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(0, device=DEV)
    acts.requires_grad_(True)
    costs = make_loss(cfg)(acts, labels, act_lens, label_lens)
    costs.sum().backward()
    c_ref, g_ref, _ = oracle.rnnt_loss(acts.detach().cpu().numpy(), labels.cpu().numpy(), act_lens.cpu().numpy(),
                                       label_lens.cpu().numpy(), cfg.blank)  # fmt: skip
    assert np.allclose(costs.detach().cpu().numpy(), c_ref, rtol=COST_RTOL)
    assert np.abs(acts.grad.cpu().numpy() - g_ref).max() < GRAD_ATOL
    # the reference's CPU path (sparse log-prob gradient + softmax Jacobian) is the same function
    c_cpu, g_cpu = oracle.rnnt_cpu_path(acts.detach().cpu().numpy(), labels.cpu().numpy(), act_lens.cpu().numpy(),
                                        label_lens.cpu().numpy(), cfg.blank, dtype=np.float32)  # fmt: skip
    assert np.allclose(costs.detach().cpu().numpy(), c_cpu, rtol=COST_RTOL)
    assert np.abs(acts.grad.cpu().numpy() - g_cpu).max() < GRAD_ATOL


def test_full_size_fused_joint():
    """The fused joint + loss at the benchmark's lattice shape (cfg 2: B=16, T=375, U=121, V=1025) with H=640: 3070
    tiles over 252 d-weight workgroups.  Checked (1) against the oracle on the smallest utterance cut out of the batch
    (costs; d f and d g rows of that utterance), and (2) through properties that hold at any size: d bias sums to
    zero over the vocabulary (every cell's gradient of the logits does), frames and label positions outside an
    utterance get exactly nothing, the gradients are linear in grad_output, and sub-batches of four utterances give the
    same costs bit for bit and the same gradients up to the rounding of their partial sums."""
    from speech_amd.joint import joint_rnnt_loss

    cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(1, device=DEV, generate_on_device=True)
    del acts
    B, T, U, V, H = cfg.B, cfg.T, cfg.U, cfg.V, 640
    gen = torch.Generator(device=DEV).manual_seed(77)
    f0 = torch.randn(B, T, H, device=DEV, generator=gen).to(torch.bfloat16)
    g0 = torch.randn(B, U, H, device=DEV, generator=gen).to(torch.bfloat16)
    W0 = torch.randn(V, H, device=DEV, generator=gen) / H**0.5
    b0 = torch.randn(V, device=DEV, generator=gen) * 0.1

    def run(scale, fused_batch_size=None):
        t = [x.clone().requires_grad_(True) for x in (f0, g0, W0, b0)]
        costs = joint_rnnt_loss(*t, labels, act_lens, label_lens, cfg.blank, fused_batch_size=fused_batch_size)
        (costs * scale).sum().backward()
        return costs.detach(), [x.grad for x in t]

    costs, (df, dg, dW, db) = run(1.0)
    assert bool(torch.isfinite(costs).all()) and bool((costs > 0).all())
    for x in (df, dg, dW, db):
        assert bool(torch.isfinite(x.float()).all())
    # (2a) a cell's gradient of the logits sums to zero over the vocabulary, so d bias does
    assert db.abs().max().item() > 1.0 and abs(db.sum().item()) <= 1e-3 * db.abs().sum().item()
    # (2b) nothing outside the utterances
    t_idx = torch.arange(T, device=DEV).view(1, T, 1)
    u_idx = torch.arange(U, device=DEV).view(1, U, 1)
    assert bool((df[(t_idx >= act_lens.view(B, 1, 1)).expand_as(df)] == 0).all())
    assert bool((dg[(u_idx > label_lens.view(B, 1, 1)).expand_as(dg)] == 0).all())
    # (2c) linear in grad_output (a power of two: exact up to the bf16 roundings' own scaling)
    costs2, (df2, dg2, dW2, db2) = run(2.0)
    assert torch.equal(costs2, costs)
    for a, b in ((df, df2), (dg, dg2), (dW, dW2), (db, db2)):
        assert (2 * a.float() - b.float()).abs().max().item() <= 2.0**-7 * b.float().abs().max().item()
    # (2d) sub-batches
    costs4, (df4, dg4, dW4, db4) = run(1.0, fused_batch_size=4)
    assert torch.equal(costs4, costs) and torch.equal(df4, df) and torch.equal(dg4, dg)
    for a, b in ((dW, dW4), (db, db4)):
        assert (a - b).abs().max().item() <= 1e-4 * a.abs().max().item()
    # (1) the smallest utterance against the oracle
    b = int((act_lens * (label_lens + 1)).argmin())
    tb, ub = int(act_lens[b]), int(label_lens[b]) + 1
    ref = oracle.joint_rnnt_loss(f0[b : b + 1, :tb].float().cpu().numpy(), g0[b : b + 1, :ub].float().cpu().numpy(),
                                 W0.cpu().numpy(), b0.cpu().numpy(), labels[b : b + 1, : ub - 1].cpu().numpy(), [tb],
                                 [ub - 1], cfg.blank)  # fmt: skip
    np.testing.assert_allclose(costs[b].item(), ref[0][0], rtol=COST_RTOL)
    for got, want in ((df[b, :tb], ref[1][0]), (dg[b, :ub], ref[2][0])):
        err = np.abs(got.float().cpu().numpy() - want).max()
        assert err <= 2.0**-6 * np.abs(want).max() + 1e-7, err
