"""GPU parity of the fused joint + RNNT loss (mi_joint_rnnt_forward / mi_joint_rnnt_backward / mi_joint_reduce_hidden
through speech_amd.joint) against oracle.joint_rnnt_loss.

Tolerances.  Costs: 1e-5 relative (the bar of the loss itself; float32 accumulation against the oracle's exact
sums of the same bf16 operands).  Gradients: the backward forms the probabilities from the fp16 copy of the logits
the forward kept (2^-11 relative on a logit) and rounds the gradient of the logits and d hidden to bf16, as the
reference's autocast backward does (roundings of 2^-9 on every term of the sums over u and t, whose terms may cancel),
so each gradient tensor is held to 2^-6 of its own largest entry."""

import numpy as np
import pytest
import torch

import oracle
from speech_amd.joint import joint_dropout_mask, joint_rnnt_forward, joint_rnnt_loss
from speech_amd import RNNTLossNumba

from gpu_utils import DEV

pytestmark = pytest.mark.gpu


def make_case(seed, B, T, U, H, V, ragged=True, scale=1.0):
    rng = np.random.RandomState(seed)
    f = torch.tensor(rng.randn(B, T, H) * scale, dtype=torch.bfloat16)
    g = torch.tensor(rng.randn(B, U, H) * scale, dtype=torch.bfloat16)
    W = torch.tensor(rng.randn(V, H) / np.sqrt(H), dtype=torch.float32)
    bias = torch.tensor(rng.randn(V) * 0.5, dtype=torch.float32)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    if ragged:
        al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
        al[0], ll[-1] = T, U - 1
    else:
        al, ll = np.full(B, T), np.full(B, U - 1)
    return f, g, W, bias, labels, al, ll


def dev_ints(*arrays):
    return [torch.tensor(np.asarray(a), dtype=torch.int64, device=DEV) for a in arrays]


def check(seed, B, T, U, H, V, lam=0.0, clamp=0.0, ragged=True, bias_on=True, weight_dtype=torch.float32,
          activation="relu"):
    f, g, W, bias, labels, al, ll = make_case(seed, B, T, U, H, V, ragged)
    rng = np.random.RandomState(seed + 1000)
    gc = (rng.rand(B) + 0.5).astype(np.float32)
    Wq = W.to(weight_dtype)
    bq = bias.to(weight_dtype) if bias_on else None
    ref = oracle.joint_rnnt_loss(f.float().numpy(), g.float().numpy(), Wq.float().numpy(),
                                 None if bq is None else bq.float().numpy(), labels, al, ll, V - 1, lam, clamp, gc,
                                 activation=activation)  # fmt: skip
    fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    Wd = Wq.to(DEV).requires_grad_(True)
    bd = None if bq is None else bq.to(DEV).requires_grad_(True)
    lab, ald, lld = dev_ints(labels, al, ll)
    costs = joint_rnnt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, lam, clamp, activation=activation)
    (costs * torch.tensor(gc, device=DEV)).sum().backward()
    torch.cuda.synchronize()
    assert costs.dtype == torch.float32 and costs.shape == (B,)
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref[0], rtol=1e-5)
    got = [fd.grad, gd.grad, Wd.grad] + ([] if bd is None else [bd.grad])
    for name, x, want in zip(("d_f", "d_g", "d_weight", "d_bias"), got, ref[1:]):
        assert x.shape == want.shape, name
        err = np.abs(x.float().cpu().numpy() - want).max()
        assert err <= 2.0**-6 * np.abs(want).max() + 1e-7, (name, err, np.abs(want).max())
    assert fd.grad.dtype == torch.bfloat16 and Wd.grad.dtype == weight_dtype
    return costs


@pytest.mark.parametrize("H", [256, 320, 384, 512, 640])
@pytest.mark.parametrize("V", [2, 37, 128, 129, 1025])
def test_small_lattices_every_vocabulary_tiling(H, V):
    check(V + H, 3, 7, 5, H, V)


def test_fastemit_and_clamp():
    check(1, 3, 9, 6, 640, 130, lam=0.01, clamp=0.05)


@pytest.mark.parametrize("activation", ["tanh", "sigmoid"])
@pytest.mark.parametrize("H,V", [(256, 37), (640, 129), (320, 1025)])
def test_tanh_and_sigmoid_joints(activation, H, V):
    """The other two activations the reference's joint accepts (modules/rnnt.py:1762-1770).  The kernel's float
    tanh / exp and the oracle's float64 ones round to different bf16 neighbours for a few hidden units in a
    hundred thousand; at these sizes that moves a cost by well under the 1e-5 bar."""
    check(V + H + len(activation), 3, 8, 5, H, V, lam=0.01, activation=activation)
    f, g, W, bias, labels, al, ll = make_case(1, 1, 2, 2, H, V)
    lab, ald, lld = dev_ints(labels, al, ll)
    with pytest.raises(ValueError, match="Unsupported activation"):  # the reference's message, modules/rnnt.py:1763
        joint_rnnt_loss(f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV), lab, ald, lld, V - 1, activation="gelu")


def test_full_lengths_no_bias_bf16_weights():
    check(2, 2, 6, 4, 640, 300, ragged=False, bias_on=False, weight_dtype=torch.bfloat16)


def test_many_tiles_per_utterance_and_tile_tails():
    # T_b * U_b of 1, 127, 128, 390 and 559 cells: a full tile, tails of 1, 6, 47 and 127 rows
    f, g, W, bias, labels, _, _ = make_case(3, 5, 130, 13, 640, 257, ragged=False)
    al, ll = np.array([1, 127, 16, 130, 43]), np.array([0, 0, 7, 2, 12])
    ref = oracle.joint_rnnt_loss(f.float().numpy(), g.float().numpy(), W.numpy(), bias.numpy(), labels, al, ll, 256)
    lab, ald, lld = dev_ints(labels, al, ll)
    fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    Wd, bd = W.to(DEV).requires_grad_(True), bias.to(DEV).requires_grad_(True)
    costs = joint_rnnt_loss(fd, gd, Wd, bd, lab, ald, lld, 256)
    costs.sum().backward()
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref[0], rtol=1e-5)
    for x, want in zip((fd.grad, gd.grad, Wd.grad, bd.grad), ref[1:]):
        assert np.abs(x.float().cpu().numpy() - want).max() <= 2.0**-6 * np.abs(want).max()
    # frames and label positions outside an utterance receive exactly nothing
    for b in range(5):
        assert torch.all(fd.grad[b, al[b] :] == 0) and torch.all(gd.grad[b, ll[b] + 1 :] == 0)


def test_forward_agrees_with_the_loss_on_materialised_logits():
    """The unfused pipeline of the reference: joint tensor first, then the loss module on it."""
    f, g, W, bias, labels, al, ll = make_case(4, 4, 30, 11, 640, 1025)
    al[1], ll[2] = 30, 10
    lab, ald, lld = dev_ints(labels, al, ll)
    fd, gd, Wd, bd = f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV)
    fused = joint_rnnt_forward(fd, gd, Wd, bd, lab, ald, lld, 1024)
    hidden = torch.relu(fd.unsqueeze(2) + gd.unsqueeze(1)).float()
    logits = hidden @ Wd.to(torch.bfloat16).float().t() + bd
    unfused = RNNTLossNumba(blank=1024, reduction='none')(logits.contiguous(), lab, ald, lld)
    np.testing.assert_allclose(fused.cpu().numpy(), unfused.cpu().numpy(), rtol=2e-5)


def test_rejects_unsupported_hidden_size_and_bad_shapes():
    lab, ald, lld = dev_ints(np.zeros((2, 2)), [3, 3], [2, 2])
    f = torch.zeros(2, 3, 192, dtype=torch.bfloat16, device=DEV)
    g = torch.zeros(2, 3, 192, dtype=torch.bfloat16, device=DEV)
    W = torch.zeros(5, 192, device=DEV)
    with pytest.raises(RuntimeError):
        joint_rnnt_forward(f, g, W, None, lab, ald, lld, 4)
    with pytest.raises(ValueError):
        joint_rnnt_forward(f, g[:, :, :64], W, None, lab, ald, lld, 4)
    with pytest.raises(RuntimeError):
        joint_rnnt_forward(f.cpu(), g.cpu(), W.cpu(), None, lab.cpu(), ald.cpu(), lld.cpu(), 4)
    with pytest.raises(TypeError):
        joint_rnnt_forward(f, g, W, None, lab, ald.int(), lld, 4)
    with pytest.raises(ValueError):
        joint_rnnt_forward(f, g, W, None, lab[:, :1], ald, lld, 4)
    with pytest.raises(ValueError):
        joint_rnnt_forward(f, g, W, None, lab, ald.cpu(), lld, 4)


def test_many_utterances():
    """More utterances than a workgroup scans linearly: the tile -> utterance search must land on the right one."""
    check(5, 70, 3, 2, 512, 19)


@pytest.mark.parametrize("p", [0.2, 0.5])
def test_dropout_mask_is_a_function_of_the_seed_and_keeps_the_right_share(p):
    a = joint_dropout_mask(3, 11, 7, 640, p, 1234, DEV)
    b = joint_dropout_mask(3, 11, 7, 640, p, 1234, DEV)
    c = joint_dropout_mask(3, 11, 7, 640, p, 1235, DEV)
    assert torch.equal(a, b) and not torch.equal(a, c)
    n = a.numel()
    kept = a.float().mean().item()
    assert abs(kept - (1 - p)) < 5 * (p * (1 - p) / n) ** 0.5 + 1e-4
    # no structure along any axis: every frame, label position and hidden unit keeps about the same share
    for dim in ((0, 2, 3), (0, 1, 3), (0, 1, 2)):
        share = a.float().mean(dim=dim)
        m = n / share.numel()
        assert (share - (1 - p)).abs().max().item() < 6 * (p * (1 - p) / m) ** 0.5
    # two seeds agree on about p^2 + (1-p)^2 of the units
    agree = (a == c).float().mean().item()
    assert abs(agree - (p * p + (1 - p) * (1 - p))) < 0.01
    assert joint_dropout_mask(2, 3, 4, 512, 0.0, 7, DEV).all()


@pytest.mark.parametrize("H,p", [(640, 0.2), (512, 0.5)])
def test_dropout_parity_with_the_exported_mask(H, p):
    B, T, U, V = 3, 9, 6, 130
    f, g, W, bias, labels, al, ll = make_case(21, B, T, U, H, V)
    seed = 987654321012345
    keep = joint_dropout_mask(B, T, U, H, p, seed, DEV).cpu().numpy()
    gc = (np.random.RandomState(3).rand(B) + 0.5).astype(np.float32)
    ref = oracle.joint_rnnt_loss(f.float().numpy(), g.float().numpy(), W.numpy(), bias.numpy(), labels, al, ll, V - 1,
                                 0.01, 0.0, gc, keep_mask=keep, dropout_p=p)  # fmt: skip
    fd, gd = f.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    Wd, bd = W.to(DEV).requires_grad_(True), bias.to(DEV).requires_grad_(True)
    lab, ald, lld = dev_ints(labels, al, ll)
    costs = joint_rnnt_loss(fd, gd, Wd, bd, lab, ald, lld, V - 1, 0.01, 0.0, dropout=p, seed=seed)
    (costs * torch.tensor(gc, device=DEV)).sum().backward()
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref[0], rtol=1e-5)
    for name, x, want in zip(("d_f", "d_g", "d_weight", "d_bias"), (fd.grad, gd.grad, Wd.grad, bd.grad), ref[1:]):
        err = np.abs(x.float().cpu().numpy() - want).max()
        assert err <= 2.0**-6 * np.abs(want).max() + 1e-7, (name, err)
    # the no-grad form sees the same mask; another seed gives other costs
    again = joint_rnnt_forward(fd, gd, Wd, bd, lab, ald, lld, V - 1, 0.01, dropout=p, seed=seed)
    other = joint_rnnt_forward(fd, gd, Wd, bd, lab, ald, lld, V - 1, 0.01, dropout=p, seed=seed + 1)
    assert torch.equal(again, costs.detach()) and not torch.equal(other, costs.detach())


def test_dropout_seed_follows_torch_manual_seed():
    f, g, W, bias, labels, al, ll = make_case(22, 2, 5, 4, 512, 40)
    lab, ald, lld = dev_ints(labels, al, ll)
    args = (f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV), lab, ald, lld, 39)
    torch.manual_seed(5)
    a = joint_rnnt_forward(*args, dropout=0.3)
    b = joint_rnnt_forward(*args, dropout=0.3)
    torch.manual_seed(5)
    c = joint_rnnt_forward(*args, dropout=0.3)
    assert torch.equal(a, c) and not torch.equal(a, b)
    with pytest.raises(ValueError):
        joint_rnnt_forward(*args, dropout=1.0)


def test_backward_leaves_what_the_forward_kept_and_serves_any_subset_of_the_inputs():
    """The backward only reads the saved logits and activations: a second backward through the same graph gives the
    same gradients bit for bit (the two product kernels and their partial sums have no atomics), and gradients of a
    subset of the inputs (only f and g: no d weight kernel; only weight and bias: no d hidden kernel, no reductions)
    equal the ones computed together."""
    f, g, W, bias, labels, al, ll = make_case(31, 4, 21, 9, 640, 300)
    lab, ald, lld = dev_ints(labels, al, ll)

    def grads(which):
        t = [f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV)]
        for i in which:
            t[i].requires_grad_(True)
        costs = joint_rnnt_loss(*t, lab, ald, lld, 299, 0.01, 0.0)
        first = torch.autograd.grad(costs.sum(), [t[i] for i in which], retain_graph=True)
        second = torch.autograd.grad(costs.sum(), [t[i] for i in which])
        for a, b in zip(first, second):
            assert torch.equal(a, b)
        return dict(zip(which, first))

    every = grads((0, 1, 2, 3))
    for subset in ((0, 1), (2, 3), (0,), (2,)):
        for i, x in grads(subset).items():
            assert torch.equal(x, every[i]), (subset, i)


def test_saved_rows_are_sized_by_the_tile_bound_and_checked():
    """The C entry points: a forward that keeps its logits needs room for every tile lattices without padding would have
    (both buffers or neither); the backward wants at least one output and its partial-sum buffers together."""
    import ctypes

    from speech_amd import _native
    from speech_amd.joint import fused

    lib = _native.lib()
    B, T, U, H, V = 3, 37, 11, 256, 70
    assert lib.mi_joint_tile_bound(B, T, U) == B * ((T * U + 127) // 128)
    assert lib.mi_joint_tile_bound(0, T, U) == 0 and lib.mi_joint_tile_bound(1 << 20, 1 << 15, 1 << 10) == 0
    f, g, W, bias, labels, al, ll = make_case(32, B, T, U, H, V)
    fd, gd, Wd, bd = f.to(DEV), g.to(DEV), W.to(DEV), bias.to(DEV)
    lab, ald, lld = dev_ints(labels, al, ll)
    ws = fused.joint_workspace(B, T, U, H, V, DEV)
    tiles = lib.mi_joint_tile_bound(B, T, U)
    NP = lib.mi_joint_padded_vocabulary(V)
    costs = torch.empty(B, device=DEV)
    logits = torch.empty(tiles * 128, NP, dtype=torch.float16, device=DEV)
    acts = torch.empty(tiles * 128, H + 16, dtype=torch.bfloat16, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def forward(lg, ac, n):
        return lib.mi_joint_rnnt_forward(
            fd.data_ptr(), gd.data_ptr(), Wd.data_ptr(), bd.data_ptr(), _native.DTYPE_F32, lab.data_ptr(), ald.data_ptr(),
            lld.data_ptr(), costs.data_ptr(), None, 0.0, 0, 0, B, T, U, H, V, V - 1, 0.0, 1, lg, ac, n, ws.data_ptr(),
            ws.numel(), stream)  # fmt: skip

    assert forward(logits.data_ptr(), acts.data_ptr(), tiles - 1) == _native.INVALID_VALUE
    assert forward(logits.data_ptr(), None, tiles) == _native.INVALID_VALUE
    assert forward(None, acts.data_ptr(), tiles) == _native.INVALID_VALUE
    assert forward(logits.data_ptr(), acts.data_ptr(), tiles) == _native.SUCCESS
    torch.cuda.synchronize()
    want = joint_rnnt_forward(fd, gd, Wd, bd, lab, ald, lld, V - 1)
    assert torch.equal(costs, want)
    # the saved logits are the logits: row r of tile order is cell (t, u) = divmod(r - first row of b, U_b)
    hidden = torch.relu(fd.unsqueeze(2) + gd.unsqueeze(1)).float()
    full = hidden @ Wd.to(torch.bfloat16).float().t() + bd
    row0 = 0
    for b in range(B):
        Tb, Ub = int(al[b]), int(ll[b]) + 1
        got = logits[row0 : row0 + Tb * Ub, :V].float().view(Tb, Ub, V)
        assert (got - full[b, :Tb, :Ub]).abs().max().item() <= 2.0**-10 * full[b, :Tb, :Ub].abs().max().item() + 1e-6
        assert torch.equal(acts[row0 : row0 + Tb * Ub, :H].view(Tb, Ub, H).float(), hidden[b, :Tb, :Ub].to(torch.bfloat16).float())
        assert torch.all(logits[row0 : row0 + Tb * Ub, V:NP] == float("-inf"))
        row0 += -(-Tb * Ub // 128) * 128
    d_hidden = torch.empty(tiles * 128, H, dtype=torch.bfloat16, device=DEV)
    slices = 4
    dw = torch.empty(slices, NP, H, device=DEV)
    db = torch.empty(slices, NP, device=DEV)

    def backward(dh, a, w, bpart, n):
        return lib.mi_joint_rnnt_backward(
            lab.data_ptr(), ald.data_ptr(), lld.data_ptr(), logits.data_ptr(), a, dh, w, bpart, n, tiles, None, 0, 1.0, B, T,
            U, H, V, V - 1, 0.0, 0.0, ws.data_ptr(), ws.numel(), stream)  # fmt: skip

    assert backward(None, None, None, None, slices) == _native.INVALID_VALUE                      # nothing wanted
    assert backward(None, None, dw.data_ptr(), db.data_ptr(), slices) == _native.INVALID_VALUE    # d weight needs the activations
    assert backward(None, acts.data_ptr(), dw.data_ptr(), None, slices) == _native.INVALID_VALUE  # and both partial buffers
    assert backward(None, acts.data_ptr(), dw.data_ptr(), db.data_ptr(), 0) == _native.INVALID_VALUE
    assert backward(d_hidden.data_ptr(), acts.data_ptr(), dw.data_ptr(), db.data_ptr(), slices) == _native.SUCCESS
    torch.cuda.synchronize()
    # the column sums of d weight's operands: d bias = sum over the cells of the gradient of the logits, which sums
    # to (1 - 1) = 0 over a cell's vocabulary without FastEmit: the whole vector sums to ~0 against entries of order 1
    bias_grad = db.sum(0)[:V]
    assert bias_grad.abs().max().item() > 0.1 and abs(bias_grad.sum().item()) < 1e-2 * bias_grad.abs().sum().item()
