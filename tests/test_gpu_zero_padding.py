"""The split gradient path: mi_transducer_zero_padding clears the padded cells of the gradient (a function of the
lengths alone, so it may run on another stream during the forward pass) and the backward call with
padding_zeroed != 0 then writes the valid rows only.  Together they must leave exactly what the one-pass backward
leaves, for every kernel family a row length maps to."""

import numpy as np
import pytest
import torch

from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV

pytestmark = pytest.mark.gpu


def make(seed, B, T, U, V, dtype):
    rng = np.random.RandomState(seed)
    acts = torch.tensor(rng.randn(B, T, U, V), dtype=torch.float32).to(dtype).to(DEV)
    labels = torch.tensor(rng.randint(0, V - 1, size=(B, U - 1)), dtype=torch.int64, device=DEV)
    al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
    al[0], ll[-1] = T, U - 1
    return acts, labels, torch.tensor(al, device=DEV), torch.tensor(ll, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [29, 257, 513, 1025, 4100, 33000])
def test_rnnt_two_step_gradient_equals_the_one_pass_gradient(V, dtype):
    B, T, U = 3, 11, 7
    acts, labels, al, ll = make(V, B, T, U, V, dtype)
    ws = rnnt.new_workspace(acts)
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    scale = torch.tensor([0.5, 1.0, 2.0], device=DEV)
    rnnt.rnnt_forward(acts, labels, al, ll, costs, V - 1, 0.01, True, ws)
    one = torch.full_like(acts, float('nan'))
    rnnt.rnnt_backward(acts, labels, al, ll, one, scale, V - 1, 0.01, 0.0, ws)
    two = torch.full_like(acts, float('nan'))
    rnnt.zero_padding(two, al, ll)
    rnnt.rnnt_backward(acts, labels, al, ll, two, scale, V - 1, 0.01, 0.0, ws, padding_zeroed=True)
    torch.cuda.synchronize()
    assert torch.isfinite(one).all()
    assert torch.equal(one, two)
    for b in range(B):
        assert torch.all(one[b, int(al[b]) :] == 0) and torch.all(one[b, :, int(ll[b]) + 1 :] == 0)


@pytest.mark.parametrize("V", [40, 1025])
def test_tdt_two_step_gradient_equals_the_one_pass_gradient(V):
    B, T, U, durations = 3, 9, 6, [0, 1, 2, 3]
    acts, labels, al, ll = make(V + 1, B, T, U, V + len(durations), torch.float32)
    ws = rnnt.new_workspace(acts, len(durations))
    costs = torch.empty(B, dtype=torch.float32, device=DEV)
    rnnt.tdt_forward(acts, labels, al, ll, costs, V - 1, durations, 0.0, 0.05, False, True, ws)
    one = torch.full_like(acts, float('nan'))
    rnnt.tdt_backward(acts, labels, al, ll, one, None, V - 1, durations, 0.0, 0.0, 0.05, False, ws)
    two = torch.full_like(acts, float('nan'))
    rnnt.zero_padding(two, al, ll)
    rnnt.tdt_backward(acts, labels, al, ll, two, None, V - 1, durations, 0.0, 0.0, 0.05, False, ws, padding_zeroed=True)
    torch.cuda.synchronize()
    assert torch.isfinite(one).all() and torch.equal(one, two)
