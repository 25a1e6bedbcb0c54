"""Joint network + RNNT loss forward in one pass over the lattice cells.

The reference computes `joint_net(f.unsqueeze(2) + g.unsqueeze(1))` -- ReLU, Linear(H -> V) -- into a
[B,T,U,V] tensor (nemo/collections/asr/modules/rnnt.py:1707-1724, :1759-1777) and hands it to the
loss (:1573-1578).  `joint_rnnt_forward` takes the joint network's inputs instead and returns the same
per-utterance costs; the logits exist only tile by tile inside the kernel (bf16 operands, float32
accumulation, as under bf16 autocast).
"""

import ctypes

import torch

from speech_amd import _native
from speech_amd.rnnt_loss.rnnt import _labels_ptr, _ptr, _require_gpu, _stream

__all__ = ["joint_rnnt_forward"]


def joint_workspace(B, T, U, H, V, device):
    nbytes = ctypes.c_size_t()
    status = _native.lib().mi_joint_workspace_bytes(B, T, U, H, V, ctypes.byref(nbytes))
    if status != _native.SUCCESS:
        raise RuntimeError(
            f"joint_rnnt_forward: unsupported shape B={B} T={T} U={U} H={H} V={V} (H must be 512 or 640)"
        )
    return torch.empty(nbytes.value, dtype=torch.uint8, device=device)


def joint_rnnt_forward(f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, workspace=None):
    """costs [B] (float32) of the RNNT loss on logits = relu(f[:, :, None] + g[:, None]) @ weight.T + bias.

    f [B,T,H], g [B,U,H] (projected encoder / prediction outputs; rounded to bf16 if they are not),
    weight [V,H] and bias [V] of the joint's last Linear (float32 or bf16), labels [B,U-1] int64,
    lengths [B] int64.  No gradient is recorded.
    """
    _require_gpu(f, "joint_rnnt_forward")
    if f.dim() != 3 or g.dim() != 3 or f.shape[0] != g.shape[0] or f.shape[2] != g.shape[2]:
        raise ValueError("f must be [B,T,H] and g [B,U,H]")
    B, T, H = f.shape
    U = g.shape[1]
    V = weight.shape[0]
    if weight.dim() != 2 or weight.shape[1] != H or (bias is not None and bias.shape != (V,)):
        raise ValueError("weight must be [V,H] and bias [V]")
    f = f.detach().to(torch.bfloat16).contiguous()
    g = g.detach().to(torch.bfloat16).contiguous()
    wdtype = torch.float32 if weight.dtype == torch.float32 else torch.bfloat16
    weight = weight.detach().to(wdtype).contiguous()
    bias = None if bias is None else bias.detach().to(wdtype).contiguous()
    device = f.device
    if workspace is None:
        workspace = joint_workspace(B, T, U, H, V, device)
    costs = torch.empty(B, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        status = _native.lib().mi_joint_rnnt_forward(
            _ptr(f), _ptr(g), _ptr(weight), _ptr(bias),
            _native.DTYPE_F32 if wdtype == torch.float32 else _native.DTYPE_BF16, _labels_ptr(labels),
            _ptr(act_lens), _ptr(label_lens), _ptr(costs), B, T, U, H, V, int(blank), float(fastemit_lambda), 1,
            _ptr(workspace), workspace.numel(), _stream(device),
        )  # fmt: skip
    _native.check_status(status, "joint_rnnt_forward")
    return costs
