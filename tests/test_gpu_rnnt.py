"""GPU parity of the RNNT loss: HIP path (through the module surface and the C ABI)
against the oracle and the reference's golden vectors.

Tolerances: the north-star bar is costs within 1e-5 relative and gradients within
1e-4 absolute; the small cases are held to the reference's own, tighter, fp32
thresholds (tests/collections/asr/numba/rnnt_loss/test_rnnt_pytorch.py).
"""

import numpy as np
import pytest
import torch

import oracle
from speech_amd import RNNTLossNumba
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, call_loss, make_lengths, to_dev

pytestmark = pytest.mark.gpu

COST_RTOL = 1e-5
GRAD_ATOL = 1e-4


def check_against_oracle(acts, labels, act_lens, label_lens, blank, lam=0.0, clamp=0.0, reduction='none',
                         cost_rtol=1e-6, grad_atol=2e-6, dtype=torch.float32):  # fmt: skip
    fn = RNNTLossNumba(blank=blank, reduction=reduction, fastemit_lambda=lam, clamp=clamp if clamp > 0 else -1)
    costs, grads = call_loss(fn, acts, labels, act_lens, label_lens, dtype=dtype)
    x = torch.as_tensor(np.asarray(acts), dtype=dtype).float().numpy()  # what the kernels actually saw
    c_ref, g_ref, _ = oracle.rnnt_loss(x, labels, act_lens, label_lens, blank, lam, clamp, num_threads=4)
    if reduction == 'sum':
        c_ref = c_ref.sum(keepdims=True)
    elif reduction == 'mean':
        c_ref = c_ref.sum(keepdims=True) / len(c_ref)
        g_ref = g_ref / x.shape[0]
    assert costs.shape == c_ref.shape
    assert np.allclose(costs, c_ref, rtol=cost_rtol, atol=0), (costs, c_ref)
    err = np.abs(grads - g_ref).max()
    assert err < grad_atol, err
    return costs, grads


@pytest.mark.parametrize("name", ["small", "small_blank_last", "medium"])
def test_golden_vectors(golden, name):
    g = golden[name]
    fn = RNNTLossNumba(blank=g["blank"], reduction='sum')
    costs, grads = call_loss(fn, g["acts"], g["labels"])
    assert np.allclose(costs, sum(g["costs"]), atol=1e-8, rtol=1e-6)
    assert np.allclose(grads, np.array(g["grads"]), atol=1e-6, rtol=1e-3)


def test_golden_clamp(golden):
    g = golden["small_clamp"]
    fn = RNNTLossNumba(blank=0, reduction='sum', clamp=g["clamp"])
    costs, grads = call_loss(fn, g["acts"], g["labels"])
    assert np.allclose(costs, g["costs"], rtol=1e-6)
    assert np.allclose(grads, np.array(g["grads"]), atol=1e-7, rtol=1e-5)


@pytest.mark.parametrize("lam", [1.0, 0.01, 0.00001])
def test_golden_fastemit_cost_and_clamp(golden, lam):
    g = golden["small"]
    fn = RNNTLossNumba(blank=0, reduction='sum', fastemit_lambda=lam, clamp=0.1)
    costs, grads = call_loss(fn, g["acts"], g["labels"])
    assert np.allclose(costs, g["costs"][0] * (1.0 + lam), rtol=1e-6)
    _, g_ref, _ = oracle.rnnt_loss(g["acts"], g["labels"], g["act_lens"], g["label_lens"], 0, lam, 0.1)
    assert np.abs(grads - g_ref).max() < 1e-6


def test_reference_seeded_random_cases():
    # shapes and seeds of test_rnnt_pytorch.py:147-149 and :328-335
    rng = np.random.RandomState(0)
    acts = rng.randn(1, 4, 3, 3)
    check_against_oracle(acts, [[1, 2]], [4], [2], 0, reduction='sum')
    for lam in [1.0, 0.01, 0.00001]:
        check_against_oracle(acts, [[1, 2]], [4], [2], 0, lam=lam, reduction='sum')
    rng = np.random.RandomState(0)
    acts = rng.randn(4, 8, 11, 5)
    labels = [
        [1, 2, 4, 3, 2, 2, 1, 1, 1, 1],
        [3, 2, 2, 3, 4, 1, 1, 1, 1, 1],
        [4, 4, 1, 2, 1, 3, 4, 3, 1, 2],
        [1, 1, 2, 1, 2, 3, 3, 1, 1, 1],
    ]
    check_against_oracle(acts, labels, [8] * 4, [10] * 4, 0, reduction='sum')


@pytest.mark.parametrize("reduction", [None, 'none', 'sum', 'mean'])
def test_reductions(reduction):
    rng = np.random.RandomState(4)
    B, T, U, V = 3, 7, 5, 6
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(1, V, size=(B, U - 1))
    red = 'none' if reduction is None else reduction
    fn = RNNTLossNumba(blank=0, reduction=reduction)
    costs, grads = call_loss(fn, acts, labels)
    c_ref, g_ref, _ = oracle.rnnt_loss(acts.astype(np.float32), labels, [T] * B, [U - 1] * B, 0)
    if red == 'none':
        assert costs.shape == (B,)
    else:
        assert costs.shape == (1,)
        c_ref = c_ref.sum(keepdims=True)
        if red == 'mean':
            c_ref, g_ref = c_ref / B, g_ref / B
    assert np.allclose(costs, c_ref, rtol=1e-6)
    assert np.abs(grads - g_ref).max() < 2e-6


def test_grad_output_is_folded_in():
    rng = np.random.RandomState(6)
    B, T, U, V = 4, 6, 4, 7
    acts = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32, device=DEV, requires_grad=True)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    lab, al, ll = to_dev(labels, [T] * B, [U - 1] * B)
    w = torch.tensor([0.5, -2.0, 0.0, 3.0], device=DEV)
    costs = RNNTLossNumba(blank=V - 1, reduction='none', clamp=0.05)(acts, lab, al, ll)
    (costs * w).sum().backward()
    _, g_ref, _ = oracle.rnnt_loss(acts.detach().cpu().numpy(), labels, [T] * B, [U - 1] * B, V - 1, 0.0, 0.05)
    g_ref = g_ref * w.cpu().numpy()[:, None, None, None]  # clamp first, then grad_output (rnnt_pytorch.py:88-92)
    assert np.abs(acts.grad.cpu().numpy() - g_ref).max() < 2e-6


def test_gradient_accumulation_through_a_shared_layer():
    # test_rnnt_pytorch.py:445-507: two losses back-propagate into one weight matrix
    torch.manual_seed(0)
    base = torch.randn(3, 5, device=DEV, requires_grad=True)
    mid1 = torch.randn(1, 4, 3, 3, device=DEV)
    mid2 = torch.randn(1, 6, 5, 3, device=DEV)
    fn = RNNTLossNumba(blank=0, reduction='sum')

    def run(mid, labels):
        acts = torch.matmul(mid, base)
        lab, al, ll = to_dev(labels, [acts.shape[1]], [len(labels[0])])
        fn(acts, lab, al, ll).sum().backward()
        _, g, _ = oracle.rnnt_loss(acts.detach().cpu().numpy(), labels, [acts.shape[1]], [len(labels[0])], 0)
        return np.einsum('btuk,btuv->kv', mid.cpu().numpy().astype(np.float64), g)

    want = run(mid1, [[1, 3]]) + run(mid2, [[1, 2, 3, 4]])
    assert np.allclose(base.grad.cpu().numpy(), want, atol=1e-5)


def test_no_grad_runs_forward_only():
    rng = np.random.RandomState(8)
    B, T, U, V = 2, 9, 6, 10
    acts = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32, device=DEV)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    lab, al, ll = to_dev(labels, [T, 5], [U - 1, 2])
    costs = RNNTLossNumba(blank=V - 1, reduction='none')(acts, lab, al, ll)
    assert not costs.requires_grad
    c_ref, _, _ = oracle.rnnt_loss(acts.cpu().numpy(), labels, [T, 5], [U - 1, 2], V - 1, want_grads=False)
    assert np.allclose(costs.cpu().numpy(), c_ref, rtol=1e-6)


@pytest.mark.parametrize("V", [3, 4, 5, 29, 129, 1025, 4097])
def test_variable_lengths_and_row_alignments(V):
    """Odd and even V give every 16-byte phase of a row start; padded cells must be exactly zero."""
    rng = np.random.RandomState(V)
    B, T, U = 5, 13, 9
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, 1, 0)
    costs, grads = check_against_oracle(acts, labels, act_lens, label_lens, V - 1, lam=0.001, clamp=0.3)
    for b in range(B):
        pad = grads[b].copy()
        pad[: act_lens[b], : label_lens[b] + 1] = 0
        assert np.all(pad == 0)


@pytest.mark.parametrize("V", [258, 300, 701, 1501, 3003, 5001, 9002, 20003, 33001])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_lengths_of_every_kernel_family(V, dtype):
    """Rows of 65..1024 vectors (128 to 1024 threads per row), of several vectors per thread, and rows
    too long for either; ragged lengths so that workgroups hold live and padded rows side by side."""
    rng = np.random.RandomState(V)
    B, T, U = 2, 5, 5
    acts = rng.randn(B, T, U, V) * 1.5
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    labels[0, 0] = V - 2
    labels[0, 1] = 0
    act_lens, label_lens = np.array([T, 3]), np.array([2, U - 1])
    half = dtype != torch.float32
    costs, grads = check_against_oracle(acts, labels, act_lens, label_lens, V - 1, lam=0.001, clamp=0.3,
                                        cost_rtol=1e-6, grad_atol=2.0**-8 if half else 2e-6,
                                        dtype=dtype)  # fmt: skip
    for b in range(B):
        pad = grads[b].copy()
        pad[: act_lens[b], : label_lens[b] + 1] = 0
        assert np.all(pad == 0)


@pytest.mark.parametrize("U", [1, 2, 64, 65, 129, 257, 600])
def test_label_axis_sizes(U):
    """U = 1 (empty transcripts), wave boundaries (64/65) and the 2, 4 and 8 cells-per-lane kernels."""
    rng = np.random.RandomState(U)
    B, T, V = 2, 11, 12
    acts = rng.randn(B, T, U, V)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens = np.array([T, 4])
    label_lens = np.array([U - 1, (U - 1) // 2])
    check_against_oracle(acts, labels, act_lens, label_lens, V - 1, lam=0.01)


def test_blank_in_the_middle_and_label_equal_to_blank():
    rng = np.random.RandomState(12)
    B, T, U, V = 2, 6, 4, 9
    acts = rng.randn(B, T, U, V)
    labels = np.array([[4, 2, 4], [1, 4, 0]])  # 4 is also the blank id
    check_against_oracle(acts, labels, [T, T], [U - 1, U - 1], 4, lam=0.2, clamp=0.0)


def test_stage_level_denominator_alphas_betas():
    """Mirror of the reference's per-kernel tests (utils/test_gpu_rnnt_kernel.py:52-209): seed 0, shape [1,5,11,3]."""
    rng = np.random.RandomState(0)
    B, T, U, V = 1, 5, 11, 3
    x = rng.randn(B, T, U, V)
    labels = np.array([[1, 1, 1, 2, 2, 2, 1, 2, 2, 1]])
    acts = torch.tensor(x, dtype=torch.float32, device=DEV)
    lab, al, ll = to_dev(labels, [T], [U - 1])
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    ws = rnnt.new_workspace(acts)
    rnnt.rnnt_forward(acts, lab, al, ll, costs, 0, 0.0, True, ws)
    denom, alphas, betas, llf, llb = [t.cpu().numpy() for t in rnnt.export_lattice(ws, al, ll, B, T, U)]
    _, _, ex = oracle.rnnt_loss(x.astype(np.float32), labels, [T], [U - 1], 0)
    assert np.abs(denom - ex["denom"]).max() < 1e-6
    assert np.abs(alphas - ex["alphas"]).mean() <= 1e-5 and np.abs(alphas - ex["alphas"]).max() < 1e-5
    assert np.abs(betas - ex["betas"]).mean() <= 1e-5 and np.abs(betas - ex["betas"]).max() < 1e-5
    assert abs(llf[0] - ex["ll_forward"][0]) < 1e-5 and abs(llb[0] - ex["ll_backward"][0]) < 1e-5
    assert abs(llf[0] - llb[0]) < 1e-5


def test_function_level_seam_fills_caller_buffers():
    rng = np.random.RandomState(14)
    B, T, U, V = 3, 8, 5, 17
    x = rng.randn(B, T, U, V).astype(np.float32)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens, label_lens = np.array([T, 6, 3]), np.array([2, U - 1, 0])
    acts = torch.tensor(x, device=DEV)
    lab, al, ll = to_dev(labels, act_lens, label_lens)
    costs = torch.zeros(B, dtype=torch.float32, device=DEV)
    grads = torch.full_like(acts, 7.0)  # the library must overwrite every element
    assert rnnt.rnnt_loss_gpu(acts, lab, al, ll, costs, grads, V - 1, 0.001, 0.0, 0) is True
    c_ref, g_ref, _ = oracle.rnnt_loss(x, labels, act_lens, label_lens, V - 1, 0.001)
    assert np.allclose(costs.cpu().numpy(), c_ref, rtol=1e-6)
    assert np.abs(grads.cpu().numpy() - g_ref).max() < 2e-6
    costs2 = torch.zeros(B, dtype=torch.float32, device=DEV)
    assert rnnt.rnnt_loss_gpu(acts, lab, al, ll, costs2, None, V - 1, 0.001, 0.0, 0) is True
    assert torch.equal(costs, costs2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_half_precision_io(dtype):
    """16-bit logits, fp32/fp64 accumulation: the oracle sees acts.float() (what the reference's wrapper
    feeds its kernels after the upcast, nemo/collections/asr/losses/rnnt.py:452-465); the gradient is
    rounded to the 16-bit type on store."""
    rng = np.random.RandomState(16)
    B, T, U, V = 3, 12, 7, 131
    acts = rng.randn(B, T, U, V) * 2
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    act_lens, label_lens = make_lengths(rng, B, T, U, 3, 1)
    eps = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    check_against_oracle(acts, labels, act_lens, label_lens, V - 1, lam=0.001, cost_rtol=1e-6, grad_atol=eps,
                         dtype=dtype)  # fmt: skip


def test_baseline_config_1_full():
    # B=4, T=50, U+1=21, V=129, blank 128, full lengths (the reference's CPU-runnable case)
    gen = torch.Generator().manual_seed(1234 + 0)
    B, T, U, V = 4, 50, 21, 129
    acts = torch.randn(B, T, U, V, generator=gen).numpy()
    labels = torch.randint(0, 128, (B, U - 1), generator=gen).numpy()
    check_against_oracle(acts, labels, [T] * B, [U - 1] * B, 128, cost_rtol=COST_RTOL, grad_atol=GRAD_ATOL)
    check_against_oracle(acts, labels, [T] * B, [U - 1] * B, 128, cost_rtol=1e-6, grad_atol=2e-6)


def test_error_behaviour_matches_reference():
    B, T, U, V = 2, 4, 3, 5
    acts = torch.zeros(B, T, U, V, device=DEV, requires_grad=True)
    lab, al, ll = to_dev(np.ones((B, U - 1)), [T, T], [U - 1, 1])
    fn = RNNTLossNumba(blank=0)
    with pytest.raises(TypeError):
        fn(acts, lab.int(), al, ll)
    with pytest.raises(ValueError):
        fn(acts.transpose(1, 2), lab, al, ll)  # not contiguous
    with pytest.raises(ValueError, match="Input length mismatch"):
        fn(acts, lab, al - 1, ll)
    with pytest.raises(ValueError, match="Output length mismatch"):
        fn(acts, lab, al, ll - 1)
    with pytest.raises(ValueError, match="Must have a length per example"):
        fn(acts, lab, al[:1], ll)
    fn.clamp = -0.5
    with pytest.raises(ValueError, match="clamp"):
        fn(acts, lab, al, ll)
    with pytest.raises(ValueError, match="must be on the device of acts"):
        RNNTLossNumba(blank=0)(acts.detach(), lab.cpu(), al, ll)


def test_loaded_library_is_the_in_tree_build():
    from speech_amd import _native

    with open("/proc/self/maps") as f:
        assert any(_native.LIB_PATH in line for line in f)


@pytest.mark.parametrize("V,dtype", [(520, torch.float32), (700, torch.float32), (1030, torch.float32), (1200, torch.float32),
                                     (1400, torch.float32), (2056, torch.float32), (4104, torch.float32),
                                     (8200, torch.float32), (1040, torch.bfloat16), (1500, torch.bfloat16),
                                     (2060, torch.bfloat16), (2500, torch.bfloat16)])  # fmt: skip
def test_vocabularies_just_past_a_power_of_two(V, dtype):
    """Row lengths that take the in-between kernel shapes: 3, 5 or 6 vectors per lane in the denominator pass, a
    third vector per thread in the gradient pass (e.g. 1024 tokens + blank + a few big blanks or durations)."""
    rng = np.random.RandomState(V)
    B, T, U = 2, 7, 5
    x = torch.tensor(rng.randn(B, T, U, V), dtype=dtype)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    al, ll = np.array([T, 4]), np.array([2, U - 1])
    acts = x.to(DEV).requires_grad_(True)
    lab, ald, lld = to_dev(labels, al, ll)
    costs = RNNTLossNumba(blank=V - 1, reduction='none', fastemit_lambda=0.01, clamp=0.3)(acts, lab, ald, lld)
    costs.sum().backward()
    c_ref, g_ref, _ = oracle.rnnt_loss(x.float().numpy(), labels, al, ll, V - 1, 0.01, 0.3)
    f32 = dtype == torch.float32
    np.testing.assert_allclose(costs.detach().float().cpu().numpy(), c_ref, rtol=1e-6 if f32 else 1e-5)
    assert np.abs(acts.grad.float().cpu().numpy() - g_ref).max() < (2e-6 if f32 else 2.0**-8)


def test_length_check_is_memoised_per_tensor_and_version():
    """The shape-vs-lengths check (rnnt_pytorch.py:628-634) is skipped only for the very tensor objects that
    already passed it, unmodified; an in-place change or another tensor is checked (and refused) again."""
    from speech_amd.rnnt_loss import rnnt_pytorch

    rng = np.random.RandomState(3)
    B, T, U, V = 2, 6, 4, 9
    acts = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32, device=DEV)
    lab, al, ll = to_dev(rng.randint(0, V - 1, size=(B, U - 1)), [T, 4], [U - 1, 2])
    fn = RNNTLossNumba(blank=V - 1, reduction='none')
    first = fn(acts, lab, al, ll)
    entry = rnnt_pytorch._validated.entry
    assert entry is not None and entry[0]() is al and entry[1]() is ll
    again = fn(acts, lab, al, ll)  # served from the memo: same result
    assert torch.equal(first, again)
    al[0] -= 1  # in place: the version moves, the check runs again and now fails
    with pytest.raises(ValueError, match="Input length mismatch"):
        fn(acts, lab, al, ll)
    al[0] += 1
    assert torch.equal(fn(acts, lab, al, ll), first)
    with pytest.raises(ValueError, match="Output length mismatch"):  # another tensor object: always checked
        fn(acts, lab, al, ll.clone() - 1)
    with pytest.raises(ValueError, match="Input length mismatch"):  # same tensors against another shape
        fn(acts[:, : T - 1].contiguous(), lab, al, ll)
