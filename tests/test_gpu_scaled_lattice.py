"""The scaled (probability-domain) RNNT lattice against the log-domain one and the oracle.

In lattice mode 2 `mi_rnnt_forward` runs the recursion on probabilities with block-wise power-of-two scaling and
returns, per utterance, to the log domain when its own checks say the range of a double was not enough.  Here:
  * ordinary logits: every utterance comes out in the scaled format, and costs, exported alphas / betas and gradients
    agree with the log-domain kernel (mode 1) far inside the north-star bar (costs 1e-5 relative, gradients 1e-4);
  * logits of growing spread (arc log-probs down to -2000): whichever format an utterance ends in, the results hold
    the oracle's float64 values at the same bar, and the widest spreads do end in the log format;
  * a lattice built to mislead a single scale per diagonal (an attractive prefix with a dead end) is caught.
"""

import numpy as np
import pytest
import torch

import oracle
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _scaled_mode():
    rnnt.set_lattice_mode(2)
    yield
    rnnt.set_lattice_mode(0)


def run(x, labels, al, ll, blank, dtype=torch.float32, lam=0.0, clamp=0.0):
    acts = torch.tensor(x, dtype=dtype, device=DEV)
    lab, ald, lld = to_dev(labels, al, ll)
    B, T, U, V = acts.shape
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    grads = torch.empty_like(acts)
    ws = rnnt.new_workspace(acts)
    ws.fill_(0xFF)  # nothing may depend on what the workspace held
    rnnt.rnnt_forward(acts, lab, ald, lld, costs, blank, lam, True, ws)
    fmt = rnnt.lattice_formats(ws, B, T, U).cpu().numpy()
    why = rnnt.lattice_diagnostics(ws, B, T, U).cpu().numpy()
    _, alphas, betas, llf, llb = [t.cpu().numpy() for t in rnnt.export_lattice(ws, ald, lld, B, T, U)]
    rnnt.rnnt_backward(acts, lab, ald, lld, grads, None, blank, lam, clamp, ws)
    torch.cuda.synchronize()
    return dict(costs=costs.cpu().numpy(), grads=grads.float().cpu().numpy(), alphas=alphas, betas=betas, llf=llf,
                llb=llb, fmt=fmt, why=why)  # fmt: skip


def case(seed, B, T, U, V, spread=1.0):
    rng = np.random.RandomState(seed)
    x = (rng.randn(B, T, U, V) * spread).astype(np.float32)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    al = rng.randint(max(1, T // 2), T + 1, size=B)
    ll = rng.randint(0, U, size=B)
    al[0], ll[0] = T, U - 1
    if B > 1:
        al[-1], ll[-1] = max(1, T // 3), 0
    return x, labels, al, ll


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,U,V", [(3, 9, 5, 11), (2, 40, 33, 29), (4, 75, 90, 37), (2, 120, 150, 40),
                                     (2, 60, 300, 17), (1, 30, 600, 9), (16, 64, 21, 1024)])  # fmt: skip
def test_scaled_against_log_domain(dtype, B, T, U, V):
    x, labels, al, ll = case(B * T + U, B, T, U, V, 2.0)
    if dtype == torch.bfloat16:
        x = torch.tensor(x).to(dtype).float().numpy()
    scaled = run(x, labels, al, ll, V - 1, dtype, lam=0.01, clamp=0.0)
    rnnt.set_lattice_mode(1)
    logd = run(x, labels, al, ll, V - 1, dtype, lam=0.01, clamp=0.0)
    assert (scaled["fmt"] == 1).all() and (logd["fmt"] == 0).all(), scaled["why"]
    np.testing.assert_allclose(scaled["costs"], logd["costs"], rtol=2e-6)
    np.testing.assert_allclose(scaled["llf"], scaled["llb"], rtol=1e-6)
    gtol = 2e-6 if dtype == torch.float32 else 2.0**-8
    assert np.abs(scaled["grads"] - logd["grads"]).max() <= gtol * max(1.0, np.abs(logd["grads"]).max())
    valid = np.zeros((B, T, U), bool)
    for b in range(B):
        valid[b, : al[b], : ll[b] + 1] = True
    for key in ("alphas", "betas"):
        d = np.abs(scaled[key] - logd[key])[valid]
        assert d.max() <= 1e-5 * max(1.0, np.abs(logd[key][valid]).max()), key
    # and the oracle, at the bar of the task
    c_ref, g_ref, _ = oracle.rnnt_loss(x, labels, al, ll, V - 1, 0.01, 0.0)
    np.testing.assert_allclose(scaled["costs"], c_ref, rtol=1e-5)
    if dtype == torch.float32:
        assert np.abs(scaled["grads"] - g_ref).max() < 1e-4


@pytest.mark.parametrize("spread", [10.0, 40.0, 120.0, 400.0])
def test_wide_logits_hold_the_oracle_in_either_format(spread):
    B, T, U, V = 4, 50, 24, 13
    x, labels, al, ll = case(int(spread), B, T, U, V, spread)
    x[1] = x[1] / spread  # one ordinary utterance among them
    got = run(x, labels, al, ll, V - 1)
    c_ref, g_ref, _ = oracle.rnnt_loss(x, labels, al, ll, V - 1, 0.0, 0.0)
    np.testing.assert_allclose(got["costs"], c_ref, rtol=1e-5)
    assert np.abs(got["grads"] - g_ref).max() < 1e-4
    assert got["fmt"][1] == 1
    if spread >= 400.0:
        assert (got["fmt"][[0, 2]] == 0).all()
    # whatever took the log route is bit-identical to the log-domain kernel
    rnnt.set_lattice_mode(1)
    logd = run(x, labels, al, ll, V - 1)
    for b in np.nonzero(got["fmt"] == 0)[0]:
        assert np.array_equal(got["costs"][b], logd["costs"][b])
        assert np.array_equal(got["grads"][b], logd["grads"][b])


def test_attractive_dead_end_is_caught():
    """Row t = 0 is cheap to walk along (labels at probability ~1) but everything that leaves it late is almost
    impossible, while the path that goes down first and right later is merely unlikely.  With one scale per
    diagonal the cheap prefix sets the scale and the true path sinks below the range of a double."""
    B, T, U, V = 1, 12, 12, 4
    blank = V - 1
    labels = np.zeros((B, U - 1), dtype=np.int64)
    x = np.zeros((B, T, U, V), dtype=np.float32)
    x[0, 0, :, 0] = 300.0        # along t = 0: label arcs certain, blank arcs at exp(-300)
    x[0, 1:, :, :] = 0.0         # elsewhere: uniform
    x[0, 0, 0, blank] = 0.0      # leaving (0,0) downwards costs exp(-300) as well
    x[0, 1:, 1:, blank] = -320.0  # once below row 0, going further down is hard except in column 0
    x[0, :, U - 1, blank] = 0.0
    x[0, :, U - 1, 0] = -300.0
    al, ll = np.array([T]), np.array([U - 1])
    got = run(x, labels, al, ll, blank)
    c_ref, g_ref, _ = oracle.rnnt_loss(x, labels, al, ll, blank, 0.0, 0.0)
    np.testing.assert_allclose(got["costs"], c_ref, rtol=1e-5)
    assert np.abs(got["grads"] - g_ref).max() < 1e-4


def test_minus_infinity_logits_take_the_log_route():
    B, T, U, V = 2, 7, 4, 6
    x, labels, al, ll = case(3, B, T, U, V)
    x[0, 2, 1, V - 1] = -np.inf  # a blank arc that cannot be taken
    got = run(x, labels, al, ll, V - 1)
    assert got["fmt"][0] == 0 and got["fmt"][1] == 1
    rnnt.set_lattice_mode(1)
    logd = run(x, labels, al, ll, V - 1)
    assert np.array_equal(got["costs"], logd["costs"], equal_nan=True)
    assert np.array_equal(got["grads"][0], logd["grads"][0], equal_nan=True)


def test_north_star_shape_scaled_against_log_domain():
    """The benchmark configuration at full size (B=16, T=375, U=121, V=1025, ragged lengths): every utterance stays in
    the scaled format and costs / gradients agree with the log-domain kernel far inside the bar of the task."""
    from speech_amd import RNNTLossNumba, synthetic

    cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(1, device=torch.device(DEV), generate_on_device=True)
    B, T, U, V = acts.shape
    loss = RNNTLossNumba(blank=cfg.blank, reduction="none", fastemit_lambda=0.001, clamp=0.0)
    out = {}
    for mode in (2, 1):
        rnnt.set_lattice_mode(mode)
        x = acts.detach().clone().requires_grad_(True)
        costs = loss(x, labels, act_lens, label_lens)
        costs.sum().backward()
        out[mode] = (costs.detach().double().cpu().numpy(), x.grad)
    # the formats the scaled run ended in, read from a workspace of its own
    rnnt.set_lattice_mode(2)
    ws = rnnt.new_workspace(acts)
    c = torch.empty(B, dtype=torch.float32, device=acts.device)
    rnnt.rnnt_forward(acts.detach(), labels, act_lens, label_lens, c, cfg.blank, 0.001, True, ws)
    assert (rnnt.lattice_formats(ws, B, T, U).cpu().numpy() == 1).all()
    np.testing.assert_allclose(out[2][0], out[1][0], rtol=1e-6)
    np.testing.assert_allclose(c.double().cpu().numpy(), out[1][0], rtol=1e-6)
    assert float((out[2][1] - out[1][1]).abs().max()) < 2e-6
