"""Joint network + RNNT loss without the [B,T,U,V] tensor.

The reference computes `joint_net(f.unsqueeze(2) + g.unsqueeze(1))` -- ReLU, Linear(H -> V) -- into a
[B,T,U,V] tensor (nemo/collections/asr/modules/rnnt.py:1707-1724, joint_net built at :1759-1777) and hands it
to the loss (:1573-1578); autograd then keeps that tensor and a gradient of the same size.  Here

  forward   one kernel forms the logits tile by tile on the matrix cores (bf16 operands, float32 accumulation: the
            arithmetic of bf16 autocast) and keeps only each cell's log-softmax denominator and its blank / label
            log-probs; the lattice kernel turns those into the costs;
  backward  the same kernel recomputes the logits and writes their gradient and the ReLU outputs as bf16, one row
            per VALID lattice cell (padded cells are never touched); two library GEMMs give d weight and d hidden,
            and a reduction kernel sums d hidden over u into d f and over t into d g.

`joint_rnnt_loss` is differentiable in f, g, weight and bias; `joint_rnnt_forward` is the no-grad form.
Limits: ReLU joint without dropout (the reference's default `jointnet.activation`), H in {512, 640}.
"""

import ctypes

import torch

from speech_amd import _native
from speech_amd.rnnt_loss.rnnt import _labels_ptr, _ptr, _require_gpu, _stream

__all__ = ["joint_rnnt_forward", "joint_rnnt_loss", "JointRNNTLoss"]


def joint_workspace(B, T, U, H, V, device):
    nbytes = ctypes.c_size_t()
    status = _native.lib().mi_joint_workspace_bytes(B, T, U, H, V, ctypes.byref(nbytes))
    if status != _native.SUCCESS:
        raise RuntimeError(
            f"joint_rnnt_forward: unsupported shape B={B} T={T} U={U} H={H} V={V} (H must be 512 or 640)"
        )
    return torch.empty(nbytes.value, dtype=torch.uint8, device=device)


def _check(f, g, weight, bias, labels, act_lens, label_lens):
    """Shapes, dtypes and devices (the checks certify_inputs makes for the loss modules, rnnt_pytorch.py:601-634)."""
    _require_gpu(f, "joint_rnnt_loss")
    if f.dim() != 3 or g.dim() != 3 or f.shape[0] != g.shape[0] or f.shape[2] != g.shape[2]:
        raise ValueError("f must be [B,T,H] and g [B,U,H]")
    B, U = f.shape[0], g.shape[1]
    if weight.dim() != 2 or weight.shape[1] != f.shape[2]:
        raise ValueError("weight must be [V,H]")
    if bias is not None and tuple(bias.shape) != (weight.shape[0],):
        raise ValueError("bias must be [V]")
    for name, t, shape in (("labels", labels, (B, U - 1)), ("act_lens", act_lens, (B,)), ("label_lens", label_lens, (B,))):
        if t.dtype != torch.int64:
            raise TypeError(f"{name} must be int64")
        if tuple(t.shape) != shape:
            raise ValueError(f"{name} must have shape {list(shape)}, got {list(t.shape)}")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    for name, t in (("g", g), ("weight", weight), ("bias", bias), ("labels", labels), ("act_lens", act_lens),
                    ("label_lens", label_lens)):  # fmt: skip
        if t is not None and t.device != f.device:
            raise ValueError(f"{name} must be on {f.device}")


def _forward(f16, g16, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda, workspace):
    B, T, H = f16.shape
    U, V = g16.shape[1], weight.shape[0]
    device = f16.device
    wdtype = torch.float32 if weight.dtype == torch.float32 else torch.bfloat16
    weight = weight.detach().to(wdtype).contiguous()
    bias = None if bias is None else bias.detach().to(wdtype).contiguous()
    costs = torch.empty(B, dtype=torch.float32, device=device)
    tiles = torch.empty(1, dtype=torch.int32, device=device)
    with torch.cuda.device(device):
        status = _native.lib().mi_joint_rnnt_forward(
            _ptr(f16), _ptr(g16), _ptr(weight), _ptr(bias),
            _native.DTYPE_F32 if wdtype == torch.float32 else _native.DTYPE_BF16, _labels_ptr(labels),
            _ptr(act_lens), _ptr(label_lens), _ptr(costs), _ptr(tiles), B, T, U, H, V, int(blank),
            float(fastemit_lambda), 1, _ptr(workspace), workspace.numel(), _stream(device),
        )  # fmt: skip
    _native.check_status(status, "joint_rnnt_forward")
    return costs, tiles


def joint_rnnt_forward(f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, workspace=None):
    """costs [B] (float32) of the RNNT loss on logits = relu(f[:, :, None] + g[:, None]) @ weight.T + bias.

    f [B,T,H], g [B,U,H] (projected encoder / prediction outputs; rounded to bf16 if they are not), weight [V,H] and
    bias [V] of the joint's last Linear (float32 or bf16), labels [B,U-1] int64, lengths [B] int64.  Nothing is
    recorded for autograd.
    """
    _check(f, g, weight, bias, labels, act_lens, label_lens)
    f16 = f.detach().to(torch.bfloat16).contiguous()
    g16 = g.detach().to(torch.bfloat16).contiguous()
    if workspace is None:
        workspace = joint_workspace(f.shape[0], f.shape[1], g.shape[1], f.shape[2], weight.shape[0], f.device)
    return _forward(f16, g16, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda, workspace)[0]


class JointRNNTLoss(torch.autograd.Function):
    """costs [B] = RNNT loss of the ReLU joint's logits, differentiable in f, g, weight, bias."""

    @staticmethod
    def forward(ctx, f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda, clamp):
        _check(f, g, weight, bias, labels, act_lens, label_lens)
        if clamp < 0:
            raise ValueError("`clamp` must be 0.0 or positive float value.")
        f16 = f.detach().to(torch.bfloat16).contiguous()
        g16 = g.detach().to(torch.bfloat16).contiguous()
        B, T, H = f16.shape
        workspace = joint_workspace(B, T, g16.shape[1], H, weight.shape[0], f.device)
        costs, tiles = _forward(f16, g16, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda, workspace)
        ctx.save_for_backward(f16, g16, weight, labels, act_lens, label_lens, tiles)
        ctx.workspace = workspace
        ctx.has_bias = bias is not None
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.in_dtypes = (f.dtype, g.dtype)
        ctx.args = (int(blank), float(fastemit_lambda), float(clamp))
        return costs

    @staticmethod
    def backward(ctx, grad_costs):
        f16, g16, weight, labels, act_lens, label_lens, tiles = ctx.saved_tensors
        blank, fastemit_lambda, clamp = ctx.args
        B, T, H = f16.shape
        U, V = g16.shape[1], weight.shape[0]
        device = f16.device
        lib = _native.lib()
        NP = lib.mi_joint_padded_vocabulary(V)
        ntiles = int(tiles.item())  # sizes the buffers below: the one host read-back of this op
        rows = ntiles * 128
        dlogits = torch.empty(rows, NP, dtype=torch.bfloat16, device=device)
        hidden = torch.empty(rows, H + 16, dtype=torch.bfloat16, device=device)  # activations, then 1, 1, 0, ...
        row_ft = torch.empty(rows, dtype=torch.int64, device=device)
        row_gu = torch.empty(rows, dtype=torch.int64, device=device)
        grad_costs = grad_costs.to(torch.float32)
        stride = 0 if grad_costs.numel() == 1 else (grad_costs.stride(0) if grad_costs.dim() else 0)
        workspace = ctx.workspace
        with torch.cuda.device(device):
            status = lib.mi_joint_rnnt_backward_logits(
                _ptr(f16), _ptr(g16), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(dlogits),
                _ptr(hidden), _ptr(row_ft), _ptr(row_gu), ntiles, _ptr(grad_costs), int(stride), 1.0, B, T, U, H, V,
                blank, fastemit_lambda, clamp, _ptr(workspace), workspace.numel(), _stream(device),
            )  # fmt: skip
        _native.check_status(status, "joint_rnnt_loss backward")
        d_weight = d_bias = d_f = d_g = None
        want_bias = ctx.has_bias and ctx.needs_input_grad[3]
        if ctx.needs_input_grad[2] or want_bias:
            # [NP, rows] x [rows, H+16], the long axis split 64 ways (rows is a multiple of 128): the library's kernels
            # for one such product leave most of the GPU idle.  Partial products and their sum are float32.  Column
            # H of the result is dlogits summed over the rows, the gradient of the bias (hidden holds ones there).
            parts = torch.bmm(dlogits.view(64, rows // 64, NP).transpose(1, 2), hidden.view(64, rows // 64, H + 16),
                              out_dtype=torch.float32)  # fmt: skip
            total = parts.sum(0)
            if ctx.needs_input_grad[2]:
                d_weight = total[:V, :H].to(weight.dtype)
            if want_bias:
                d_bias = total[:V, H].to(ctx.bias_dtype)
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            # the forward call's packed weights [NP, H+16] bf16, read in place (their padded rows are zero)
            packed, prow, pitch = ctypes.c_void_p(), ctypes.c_int(), ctypes.c_int()
            status = lib.mi_joint_packed_weights(
                _ptr(workspace), workspace.numel(), B, T, U, H, V, ctypes.byref(packed), ctypes.byref(prow),
                ctypes.byref(pitch),
            )  # fmt: skip
            _native.check_status(status, "joint_rnnt_loss backward")
            off = packed.value - workspace.data_ptr()
            w_packed = workspace[off : off + prow.value * pitch.value * 2].view(torch.bfloat16)
            w_packed = w_packed.view(prow.value, pitch.value)[:, :H]
            d_hidden = torch.mm(dlogits, w_packed)  # [rows, H] bf16
            want_f, want_g = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
            d_f32 = torch.empty(B, T, H, dtype=torch.float32, device=device) if want_f else None
            d_g32 = torch.empty(B, U, H, dtype=torch.float32, device=device) if want_g else None
            with torch.cuda.device(device):
                status = lib.mi_joint_reduce_hidden(
                    _ptr(d_hidden), _ptr(f16), _ptr(g16), _ptr(act_lens), _ptr(label_lens), _ptr(d_f32), _ptr(d_g32), ntiles,
                    B, T, U, H, V, _ptr(workspace), workspace.numel(), _stream(device),
                )  # fmt: skip
            _native.check_status(status, "joint_rnnt_loss backward")
            d_f = None if d_f32 is None else d_f32.to(ctx.in_dtypes[0])
            d_g = None if d_g32 is None else d_g32.to(ctx.in_dtypes[1])
        ctx.workspace = None
        return d_f, d_g, d_weight, d_bias, None, None, None, None, None, None


def joint_rnnt_loss(f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda=0.0, clamp=0.0):
    """Per-utterance RNNT costs [B] of the joint's logits, with gradients to f, g, weight and bias."""
    return JointRNNTLoss.apply(f, g, weight, bias, labels, act_lens, label_lens, blank, fastemit_lambda, clamp)
