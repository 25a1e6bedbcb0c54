"""The entry point that takes no workspace (mi_rnnt_loss_static): the lattice state lives in a device array built
into the library.  Called through the C ABI, its costs and gradients must equal those of mi_rnnt_loss on a
caller-owned workspace bit for bit -- on two calls in a row, the second on a smaller input, so that what the first
call left in the shared array is there to be (wrongly) picked up -- and a shape beyond the built-in size must be
refused without launching anything."""

import ctypes

import numpy as np
import pytest
import torch

from speech_amd import _native
from speech_amd.rnnt_loss import rnnt

from gpu_utils import DEV, to_dev

pytestmark = pytest.mark.gpu


def _case(seed, B, T, U, V, dtype):
    rng = np.random.RandomState(seed)
    x = torch.tensor(rng.randn(B, T, U, V) * 2.0, dtype=dtype, device=DEV)
    labels = rng.randint(0, V - 1, size=(B, U - 1))
    al, ll = rng.randint(1, T + 1, size=B), rng.randint(0, U, size=B)
    al[0], ll[-1] = T, U - 1
    return (x,) + to_dev(labels, al, ll)


def _both(x, lab, al, ll, lam, clamp, riders=_native.RIDERS_AUTO, riders_ref=_native.RIDERS_AUTO):
    lib = _native.lib()
    B, T, U, V = x.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    code = rnnt._dtype_code(x)
    scale = torch.linspace(0.5, 1.5, B, device=DEV)
    ws = rnnt.new_workspace(x)
    costs_ref = torch.full((B,), float("nan"), device=DEV)
    grads_ref = torch.full_like(x, float("nan"))
    st = lib.mi_rnnt_loss(x.data_ptr(), code, lab.data_ptr() if lab.numel() else None, al.data_ptr(), ll.data_ptr(),
                          costs_ref.data_ptr(), grads_ref.data_ptr(), scale.data_ptr(), 1, 0.5, B, T, U, V, V - 1, lam,
                          clamp, riders_ref, ws.data_ptr(), ws.numel(), stream)  # fmt: skip
    assert st == _native.SUCCESS
    costs = torch.full((B,), float("nan"), device=DEV)
    grads = torch.full_like(x, float("nan"))
    st = lib.mi_rnnt_loss_static(x.data_ptr(), code, lab.data_ptr() if lab.numel() else None, al.data_ptr(),
                                 ll.data_ptr(), costs.data_ptr(), grads.data_ptr(), scale.data_ptr(), 1, 0.5, B, T, U,
                                 V, V - 1, lam, clamp, riders, stream)  # fmt: skip
    assert st == _native.SUCCESS
    torch.cuda.synchronize()
    assert torch.isfinite(costs_ref).all() and torch.isfinite(grads_ref.float()).all()
    assert torch.equal(costs, costs_ref)
    assert torch.equal(grads, grads_ref)
    return grads


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_workspace_entry_point_matches_the_workspace_one(dtype):
    assert _native.lib().mi_transducer_init() == _native.SUCCESS
    _both(*_case(1, 5, 40, 23, 1025, dtype), 0.01, 0.5)   # first call
    _both(*_case(2, 3, 17, 9, 300, dtype), 0.0, 0.0)      # second call, smaller: other layout inside the same array
    _both(*_case(3, 2, 9, 4, 37, dtype), 0.01, 0.0)       # and the short-row kernels (coefficient records)


def test_static_workspace_entry_point_with_riders():
    """The lattice launch of the built-in workspace carries riders (mailbox, record and all inside the device array):
    ragged lengths and a lattice long enough for them to fill something, held to the workspace entry point WITHOUT
    riders, bit for bit, twice in a row (the second call finds the first call's record in the array)."""
    assert _native.lib().mi_transducer_init() == _native.SUCCESS
    for seed, (B, T, U, V) in ((5, (6, 300, 40, 1025)), (6, (4, 150, 33, 513))):
        x, lab, al, ll = _case(seed, B, T, U, V, torch.float32)
        al[1], al[2] = max(1, T // 8), T // 2
        assert _native.workspace_bytes(B, T, U) <= _native.STATIC_WORKSPACE_BYTES
        grads = _both(x, lab, al, ll, 0.01, 0.0, riders=_native.RIDERS_ON, riders_ref=_native.RIDERS_OFF)
        t = torch.arange(T, device=DEV).view(1, T, 1)
        u = torch.arange(U, device=DEV).view(1, 1, U)
        padded = (t >= al.view(B, 1, 1)) | (u > ll.view(B, 1, 1))
        assert padded.any() and (grads[padded] == 0).all()


def test_static_workspace_entry_point_forward_only_and_limits():
    lib = _native.lib()
    x, lab, al, ll = _case(4, 3, 12, 6, 70, torch.float32)
    B, T, U, V = x.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    costs = torch.zeros(B, device=DEV)
    want = torch.zeros(B, device=DEV)
    rnnt.rnnt_loss_gpu(x, lab, al, ll, want, None, V - 1, 0.0, 0.0, 0)
    assert rnnt.rnnt_loss_static(x, lab, al, ll, costs, None, V - 1, 0.0, 0.0) is True
    assert torch.equal(costs, want)
    # one past the built-in size: refused by the size check alone, before any pointer is looked at
    need = _native.workspace_bytes(64, 1000, 200)
    assert need > _native.STATIC_WORKSPACE_BYTES
    st = lib.mi_rnnt_loss_static(x.data_ptr(), 0, lab.data_ptr(), al.data_ptr(), ll.data_ptr(), costs.data_ptr(), None,
                                 None, 0, 1.0, 64, 1000, 200, V, V - 1, 0.0, 0.0, _native.RIDERS_AUTO, stream)  # fmt: skip
    assert st == _native.TOO_LARGE
    with pytest.raises(RuntimeError, match="built into the library"):
        _native.check_status(st, "rnnt_loss_static")
    assert lib.mi_rnnt_loss_static(x.data_ptr(), 0, lab.data_ptr(), al.data_ptr(), ll.data_ptr(), costs.data_ptr(), None,
                                   None, 0, 1.0, 0, T, U, V, V - 1, 0.0, 0.0, _native.RIDERS_AUTO, stream) == _native.INVALID_VALUE  # fmt: skip
    assert lib.mi_rnnt_loss_static(x.data_ptr(), 0, lab.data_ptr(), al.data_ptr(), ll.data_ptr(), costs.data_ptr(), None,
                                   None, 0, 1.0, B, T, U, V, V - 1, 0.0, 0.0, 7, stream) == _native.INVALID_VALUE  # fmt: skip
