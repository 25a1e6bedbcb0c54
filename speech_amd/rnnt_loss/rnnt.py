"""Function-level seam of the transducer loss on MI355X.

Mirrors nemo/collections/asr/parts/numba/rnnt_loss/rnnt.py: `rnnt_loss_gpu`
(:138-236) and `tdt_loss_gpu` (:239-363) fill caller-owned `costs` / `grads`
in place and return True; a non-success status becomes RuntimeError.  Below
them the work is done by libmi_transducer.so on torch's current stream.  The
split `*_forward` / `*_backward` functions are what the autograd Functions in
rnnt_pytorch.py use: the gradient is produced in backward with grad_output
folded in, instead of being stored in forward and rescaled later.

Differences a caller can see:
  * nothing blocks the host (the reference ends with stream.synchronize(),
    utils/cuda_utils/gpu_rnnt.py:229);
  * besides `tdt_loss_gpu` (the reference's operands: token logits and
    duration log-probs in two tensors) there is `combined_tdt_loss_gpu`, which
    takes the combined [B,T,U,V+D] logits and returns the gradient w.r.t. them
    (the kernels do the split and the duration log-softmax that
    TDTLossNumba.forward does with torch ops, rnnt_pytorch.py:564-568);
  * these functions run on the GPU only (the module-level RNNT loss has a CPU path of its own).
"""

import ctypes
import random

import torch

from speech_amd import _native

_DTYPE_CODE = {
    torch.float32: _native.DTYPE_F32,
    torch.bfloat16: _native.DTYPE_BF16,
    torch.float16: _native.DTYPE_F16,
}


def _dtype_code(t):
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"acts must be float32, bfloat16 or float16, got {t.dtype}") from None


def _require_gpu(t, what):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: this build runs on the GPU only; got a tensor on {t.device}")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _labels_ptr(labels):
    # an empty [B,0] label matrix (U == 1) has no storage to point at
    return _ptr(labels) if labels.numel() > 0 else None


def _durations_array(durations):
    arr = (ctypes.c_int32 * len(durations))(*[int(d) for d in durations])
    return arr, ctypes.cast(arr, ctypes.c_void_p)


def _check_prefill(acts, prefill_grads):
    if prefill_grads is None:
        return
    if prefill_grads.shape != acts.shape or prefill_grads.dtype != acts.dtype or prefill_grads.device != acts.device:
        raise ValueError("prefill_grads must have the shape, dtype and device of acts")
    if not prefill_grads.is_contiguous():
        raise ValueError("prefill_grads must be contiguous")


def new_workspace(acts, num_durations=0):
    """Scratch for one call (replaces torch.zeros(get_workspace_size(...)), rnnt.py:182-189; not zero-filled)."""
    B, T, U = acts.shape[:3]
    nbytes = _native.workspace_bytes(B, T, U, num_durations)
    return torch.empty(nbytes, dtype=torch.uint8, device=acts.device)


def length_maxima(act_lens, label_lens, out=None):
    """int64[2] = (max(act_lens), max(label_lens)), enqueued on the current stream.  `out` may be a
    pinned host tensor: the kernel then writes the two values straight into host memory (pinned
    allocations are mapped into the device's address space), which saves the copy back."""
    _require_gpu(act_lens, "length_maxima")
    if out is None:
        out = torch.empty(2, dtype=torch.int64, device=act_lens.device)
    elif out.dtype != torch.int64 or out.numel() != 2 or not (out.is_cuda or out.is_pinned()):
        raise ValueError("length_maxima: out must be an int64[2] device or pinned host tensor")
    with torch.cuda.device(act_lens.device):
        status = _native.lib().mi_transducer_length_maxima(
            _ptr(act_lens), _ptr(label_lens), act_lens.shape[0], _ptr(out), _stream(act_lens.device)
        )
    _native.check_status(status, "length_maxima")
    return out


def zero_padding(grads, act_lens, label_lens):
    """Zero-fill the padded cells of grads [B,T,U,V(+D)] on the CURRENT stream (nothing else is written)."""
    _require_gpu(grads, "zero_padding")
    B, T, U, VD = grads.shape
    with torch.cuda.device(grads.device):
        status = _native.lib().mi_transducer_zero_padding(
            _ptr(grads), _dtype_code(grads), _ptr(act_lens), _ptr(label_lens), B, T, U, VD, _stream(grads.device)
        )
    _native.check_status(status, "zero_padding")


def denominators(acts, labels, act_lens, label_lens, blank, workspace, num_durations=0):
    """First stage of a forward call: log-softmax denominators and gathered arc log-probs into workspace."""
    _require_gpu(acts, "denominators")
    B, T, U, VD = acts.shape
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_transducer_denominators(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), B, T, U,
            VD - num_durations, num_durations, int(blank), _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    _native.check_status(status, "Could not calculate forward scores")


def rnnt_lattice(act_lens, label_lens, costs, B, T, U, fastemit_lambda, with_betas, workspace, num_durations=0):
    """Second stage: alpha (and beta) recursions and costs from what denominators() left in workspace."""
    with torch.cuda.device(workspace.device):
        status = _native.lib().mi_rnnt_lattice(
            _ptr(act_lens), _ptr(label_lens), _ptr(costs), B, T, U, num_durations, float(fastemit_lambda),
            int(bool(with_betas)), _ptr(workspace), workspace.numel(), _stream(workspace.device),
        )  # fmt: skip
    _native.check_status(status, "Could not calculate forward scores")


def tdt_lattice(act_lens, label_lens, costs, B, T, U, durations, fastemit_lambda, sigma, with_betas, workspace):
    keep, dur_ptr = _durations_array(durations)
    with torch.cuda.device(workspace.device):
        status = _native.lib().mi_tdt_lattice(
            _ptr(act_lens), _ptr(label_lens), _ptr(costs), B, T, U, len(durations), dur_ptr, float(fastemit_lambda),
            float(sigma), int(bool(with_betas)), _ptr(workspace), workspace.numel(), _stream(workspace.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate forward scores")


def rnnt_forward(acts, labels, act_lens, label_lens, costs, blank, fastemit_lambda, with_betas, workspace,
                 prefill_grads=None):
    """prefill_grads: the buffer (shape and dtype of acts) that the backward call of this forward call will write the
    gradient into, or None.  While the lattice recursion runs, extra workgroups of its launch zero-fill the padded
    cells of that buffer as far as they get; rnnt_backward(..., padding_zeroed=2) then skips what they did."""
    _require_gpu(acts, "rnnt_forward")
    B, T, U, V = acts.shape
    _check_prefill(acts, prefill_grads)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_rnnt_forward(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(costs),
            B, T, U, V, int(blank), float(fastemit_lambda), int(bool(with_betas)), _ptr(prefill_grads),
            _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    _native.check_status(status, "Could not calculate forward scores")


def rnnt_backward(
    acts, labels, act_lens, label_lens, grads, grad_scale, blank, fastemit_lambda, clamp, workspace,
    grad_scale_stride=1, grad_mul=1.0, padding_zeroed=False,
):  # fmt: skip
    """grad_scale: device float32 tensor read as grad_scale[b * grad_scale_stride] (or None); every gradient is
    additionally multiplied by the host scalar grad_mul.  padding_zeroed: zero_padding() already ran on grads
    and the current stream waits for it (1), or the forward call was given grads as prefill_grads (2)."""
    _require_gpu(acts, "rnnt_backward")
    B, T, U, V = acts.shape
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_rnnt_backward(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(grads),
            _ptr(grad_scale), int(grad_scale_stride), float(grad_mul), int(padding_zeroed), B, T, U, V, int(blank),
            float(fastemit_lambda), float(clamp), _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    _native.check_status(status, "Could not calculate gradients")


def tdt_forward(
    acts, labels, act_lens, label_lens, costs, blank, durations, fastemit_lambda, sigma, use_plain_rnnt, with_betas,
    workspace, prefill_grads=None,
):  # fmt: skip
    """prefill_grads: as for rnnt_forward."""
    _require_gpu(acts, "tdt_forward")
    B, T, U, VD = acts.shape
    _check_prefill(acts, prefill_grads)
    D = len(durations)
    keep, dur_ptr = _durations_array(durations)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_tdt_forward(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(costs),
            B, T, U, VD - D, D, dur_ptr, int(blank), float(fastemit_lambda), float(sigma), int(bool(use_plain_rnnt)),
            int(bool(with_betas)), _ptr(prefill_grads), _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate forward scores")


def tdt_backward(
    acts, labels, act_lens, label_lens, grads, grad_scale, blank, durations, fastemit_lambda, clamp, sigma,
    use_plain_rnnt, workspace, grad_scale_stride=1, grad_mul=1.0, padding_zeroed=False,
):  # fmt: skip
    _require_gpu(acts, "tdt_backward")
    B, T, U, VD = acts.shape
    D = len(durations)
    keep, dur_ptr = _durations_array(durations)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_tdt_backward(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(grads),
            _ptr(grad_scale), int(grad_scale_stride), float(grad_mul), int(padding_zeroed), B, T, U, VD - D, D,
            dur_ptr, int(blank), float(fastemit_lambda), float(clamp), float(sigma), int(bool(use_plain_rnnt)),
            _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate gradients")


def multiblank_forward(
    acts, labels, act_lens, label_lens, costs, blank, big_blank_durations, fastemit_lambda, sigma, with_betas, workspace,
    prefill_grads=None,
):  # fmt: skip
    """prefill_grads: as for rnnt_forward."""
    _require_gpu(acts, "multiblank_forward")
    B, T, U, V = acts.shape
    _check_prefill(acts, prefill_grads)
    keep, dur_ptr = _durations_array(big_blank_durations)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_multiblank_forward(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(costs),
            B, T, U, V, len(big_blank_durations), dur_ptr, int(blank), float(fastemit_lambda), float(sigma),
            int(bool(with_betas)), _ptr(prefill_grads), _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate forward scores")


def multiblank_backward(
    acts, labels, act_lens, label_lens, grads, grad_scale, blank, big_blank_durations, fastemit_lambda, clamp, sigma,
    workspace, grad_scale_stride=1, grad_mul=1.0, padding_zeroed=0,
):  # fmt: skip
    _require_gpu(acts, "multiblank_backward")
    B, T, U, V = acts.shape
    keep, dur_ptr = _durations_array(big_blank_durations)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_multiblank_backward(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(grads),
            _ptr(grad_scale), int(grad_scale_stride), float(grad_mul), int(padding_zeroed), B, T, U, V,
            len(big_blank_durations), dur_ptr,
            int(blank), float(fastemit_lambda), float(clamp), float(sigma), _ptr(workspace), workspace.numel(),
            _stream(acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate gradients")


def export_lattice(workspace, act_lens, label_lens, B, T, U, num_durations=0):
    """(denom, alphas, betas, ll_forward, ll_backward) as plain float32 tensors, for stage-level checks."""
    dev = workspace.device
    denom = torch.empty(B, T, U, dtype=torch.float32, device=dev)
    alphas = torch.empty_like(denom)
    betas = torch.empty_like(denom)
    llf = torch.empty(B, dtype=torch.float32, device=dev)
    llb = torch.empty_like(llf)
    with torch.cuda.device(dev):
        status = _native.lib().mi_transducer_export_lattice(
            _ptr(workspace), workspace.numel(), _ptr(act_lens), _ptr(label_lens), B, T, U, num_durations,
            _ptr(denom), _ptr(alphas), _ptr(betas), _ptr(llf), _ptr(llb), _stream(dev),
        )  # fmt: skip
    _native.check_status(status, "export_lattice")
    return denom, alphas, betas, llf, llb


def prefilled_cells(workspace, act_lens, label_lens, B, T, U, row_elems, elem_bytes, num_durations=0):
    """bool[B, T, U]: the padded cells whose gradient rows the riders of the last forward call with prefill_grads
    zero-filled, read from the record in `workspace`.  row_elems = V + D of the gradient rows."""
    off, words, rows = ctypes.c_size_t(0), ctypes.c_int(0), ctypes.c_int(0)
    status = _native.lib().mi_transducer_prefill_record(
        B, T, U, num_durations, int(row_elems) * int(elem_bytes), ctypes.byref(off), ctypes.byref(words), ctypes.byref(rows)
    )
    _native.check_status(status, "prefill_record")
    record = workspace[off.value : off.value + 4 * words.value].view(torch.int32).to(torch.int64)
    dev = workspace.device
    per_frame = (U + rows.value - 1) // rows.value
    u = torch.arange(U, device=dev)
    item = torch.arange(B * T, device=dev).view(B, T, 1) * per_frame + (u // rows.value).view(1, 1, U)
    done = torch.div(item, words.value, rounding_mode="floor") < record[item % words.value]
    t = torch.arange(T, device=dev).view(1, T, 1)
    padded = (t >= act_lens.view(B, 1, 1)) | (u.view(1, 1, U) > label_lens.view(B, 1, 1))
    return done & padded


def _require_cpu_f32(t, what):
    if t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"{what} must be a contiguous float32 CPU tensor")


def cpu_workspace(acts):
    B, T, U = acts.shape[:3]
    return torch.empty(_native.cpu_workspace_bytes(B, T, U) // 8 + 1, dtype=torch.float64)


def rnnt_cpu_forward(acts, labels, act_lens, label_lens, costs, blank, fastemit_lambda, workspace, num_threads=0):
    """costs (float32 [B]) of float32 CPU logits [B,T,U,V]; `workspace` (cpu_workspace) keeps the lattice for
    rnnt_cpu_backward.  The library applies the log_softmax the reference's module applies with torch."""
    _require_cpu_f32(acts, "acts")
    B, T, U, V = acts.shape
    status = _native.cpu_lib().mi_rnnt_cpu_forward(
        _ptr(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(costs), B, T, U, V, int(blank),
        float(fastemit_lambda), _ptr(workspace), workspace.numel() * 8, int(num_threads),
    )  # fmt: skip
    _native.check_status(status, "Could not calculate forward scores")


def rnnt_cpu_backward(
    acts, labels, act_lens, label_lens, grads, grad_scale, blank, fastemit_lambda, clamp, workspace,
    grad_scale_stride=1, grad_mul=1.0, wrt_log_probs=False, num_threads=0,
):  # fmt: skip
    """Gradient w.r.t. the logits (wrt_log_probs: the reference's sparse gradient w.r.t. the log-probs), scaled per
    utterance by grad_scale[b * stride] * grad_mul and then clamped (clamp > 0)."""
    _require_cpu_f32(acts, "acts")
    _require_cpu_f32(grads, "grads")
    B, T, U, V = acts.shape
    status = _native.cpu_lib().mi_rnnt_cpu_backward(
        _ptr(acts), _labels_ptr(labels), _ptr(act_lens), _ptr(label_lens), _ptr(grads), _ptr(grad_scale),
        int(grad_scale_stride), float(grad_mul), B, T, U, V, int(blank), float(fastemit_lambda), float(clamp),
        int(bool(wrt_log_probs)), _ptr(workspace), workspace.numel() * 8, int(num_threads),
    )  # fmt: skip
    _native.check_status(status, "Could not calculate gradients")


def rnnt_loss_cpu(
    acts, labels, input_lengths, label_lengths, costs, grads, blank_label, fastemit_lambda, clamp, num_threads=0
):
    """Drop-in for rnnt.py:39-135: `acts` are LOG-PROBS (the module has applied log_softmax, rnnt_pytorch.py:435);
    costs (float32 [B]) and grads (or None: forward only) are filled in place, grads with the sparse gradient
    w.r.t. the log-probs that CPURNNT leaves (cpu_rnnt.py:327-343; `clamp` is not applied here either: the
    reference clamps in its autograd hook).  num_threads < 0: every core (rnnt.py:83-86)."""
    del clamp
    _require_cpu_f32(acts, "acts")
    if costs.dtype != torch.float32 or costs.is_cuda:
        raise TypeError("costs must be a float32 CPU tensor")
    workspace = cpu_workspace(acts)  # raises the reference's RuntimeError for non-positive dims
    threads = 0 if num_threads < 0 else max(1, int(num_threads))
    rnnt_cpu_forward(acts, labels, input_lengths, label_lengths, costs, blank_label, fastemit_lambda, workspace, threads)
    if grads is not None:
        rnnt_cpu_backward(acts, labels, input_lengths, label_lengths, grads, None, blank_label, fastemit_lambda, 0.0,
                          workspace, wrt_log_probs=True, num_threads=threads)  # fmt: skip
    return True


def _riders_code(riders):
    """None: by the size of the gradient (32 MiB and more); True / False: with / without riders in the lattice launch."""
    return _native.RIDERS_AUTO if riders is None else (_native.RIDERS_ON if riders else _native.RIDERS_OFF)


def rnnt_loss_gpu(
    acts, labels, input_lengths, label_lengths, costs, grads, blank_label, fastemit_lambda, clamp, num_threads=0,
    *, riders=None,
):  # fmt: skip
    """Drop-in for rnnt.py:138-236: costs (float32 [B]) and grads (or None) are filled in place.  `riders` (not in
    the reference; same results either way): see _riders_code."""
    del num_threads  # an OpenMP knob of the reference's CPU path; unused on the GPU there too
    _require_gpu(acts, "rnnt_loss_gpu")
    B, T, U, V = acts.shape
    workspace = new_workspace(acts)  # raises the reference's RuntimeError for non-positive dims
    if costs.dtype != torch.float32:
        raise TypeError("costs must be float32")
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_rnnt_loss(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(input_lengths), _ptr(label_lengths), _ptr(costs),
            _ptr(grads), None, 0, 1.0, B, T, U, V, int(blank_label), float(fastemit_lambda), float(clamp),
            _riders_code(riders), _ptr(workspace), workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    _native.check_status(status, "Could not calculate forward scores")
    # the caching allocator frees `workspace` in stream order, so it may go out of scope here
    return True


def tdt_loss_gpu(
    label_acts, duration_acts, labels, input_lengths, label_lengths, costs, label_grads, duration_grads, blank_label,
    durations, fastemit_lambda, clamp, num_threads, sigma, omega, *, riders=None,
):  # fmt: skip
    """Drop-in for rnnt.py:239-363, argument for argument: label_acts [B,T,U,V] are raw token logits,
    duration_acts [B,T,U,D] duration log-probs; costs [B], label_grads [B,T,U,V] (gradient w.r.t. the token
    logits) and duration_grads [B,T,U,D] (gradient w.r.t. the duration log-probs, gpu_rnnt_kernel.py:1328-1341) are
    filled in place; label_grads None means forward only (rnnt.py:336-345).  With probability omega the call takes
    the plain RNNT kernels and leaves duration_grads zero; the draw is random.uniform(0, 1) as in gpu_rnnt.py:606.
    costs may be float32 or, as the reference allocates it (rnnt_pytorch.py:145), of the dtype of the logits."""
    del num_threads
    _require_gpu(label_acts, "tdt_loss_gpu")
    if label_acts.dtype != duration_acts.dtype or label_acts.shape[:3] != duration_acts.shape[:3]:
        raise ValueError("label_acts and duration_acts must share dtype and their first three dimensions")
    if not (label_acts.is_contiguous() and duration_acts.is_contiguous()):
        raise ValueError("label_acts and duration_acts must be contiguous")
    B, T, U, V = label_acts.shape
    D = len(durations)
    if duration_acts.shape[3] != D:
        raise ValueError(f"duration_acts must hold {D} entries per cell, got {duration_acts.shape[3]}")
    if (label_grads is None) != (duration_grads is None):
        raise ValueError("label_grads and duration_grads are given together or not at all")
    workspace = new_workspace(label_acts, D)
    costs32 = costs if costs.dtype == torch.float32 else torch.empty(B, dtype=torch.float32, device=costs.device)
    use_plain_rnnt = random.uniform(0, 1) < omega
    keep, dur_ptr = _durations_array(durations)
    with torch.cuda.device(label_acts.device):
        status = _native.lib().mi_tdt_split_loss(
            _ptr(label_acts), _ptr(duration_acts), _dtype_code(label_acts), _labels_ptr(labels), _ptr(input_lengths),
            _ptr(label_lengths), _ptr(costs32), _ptr(label_grads), _ptr(duration_grads), None, 0, 1.0, B, T, U, V, D,
            dur_ptr, int(blank_label), float(fastemit_lambda), float(clamp), float(sigma), int(use_plain_rnnt),
            _riders_code(riders), _ptr(workspace), workspace.numel(), _stream(label_acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate forward scores")
    if costs32 is not costs:
        costs.copy_(costs32)
    return True


def rnnt_loss_static(acts, labels, input_lengths, label_lengths, costs, grads, blank_label, fastemit_lambda, clamp,
                     *, riders=None):
    """rnnt_loss_gpu for callers that must not allocate (HIP graph capture, serving loops): same results, but the
    lattice state lives in a 64 MiB device array built into the library instead of a workspace tensor, so this
    function creates no tensor at all.  Shapes whose workspace is larger raise RuntimeError.  Calls on one GPU
    share that array: they must not overlap in time (one stream, or the caller orders them)."""
    _require_gpu(acts, "rnnt_loss_static")
    B, T, U, V = acts.shape
    if costs.dtype != torch.float32:
        raise TypeError("costs must be float32")
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_rnnt_loss_static(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(input_lengths), _ptr(label_lengths), _ptr(costs),
            _ptr(grads), None, 0, 1.0, B, T, U, V, int(blank_label), float(fastemit_lambda), float(clamp),
            _riders_code(riders), _stream(acts.device),
        )  # fmt: skip
    _native.check_status(status, "rnnt_loss_static")
    return True


def combined_tdt_loss_gpu(
    acts, labels, input_lengths, label_lengths, costs, grads, blank_label, durations, fastemit_lambda, clamp,
    num_threads=0, sigma=0.0, use_plain_rnnt=False, *, riders=None,
):  # fmt: skip
    """TDT on the COMBINED [B,T,U,V+D] logits (what TDTLossNumba.forward receives, rnnt_pytorch.py:554-583): the
    split, the duration log_softmax and its backward happen in the kernels, and grads is w.r.t. the combined
    logits.  costs is float32 [B].  The caller decides the omega branch (use_plain_rnnt)."""
    del num_threads
    _require_gpu(acts, "combined_tdt_loss_gpu")
    B, T, U, VD = acts.shape
    D = len(durations)
    workspace = new_workspace(acts, D)
    if costs.dtype != torch.float32:
        raise TypeError("costs must be float32")
    keep, dur_ptr = _durations_array(durations)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_tdt_loss(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(input_lengths), _ptr(label_lengths), _ptr(costs),
            _ptr(grads), None, 0, 1.0, B, T, U, VD - D, D, dur_ptr, int(blank_label), float(fastemit_lambda),
            float(clamp), float(sigma), int(bool(use_plain_rnnt)), _riders_code(riders), _ptr(workspace),
            workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate forward scores")
    return True


def multiblank_rnnt_loss_gpu(
    acts, labels, input_lengths, label_lengths, costs, grads, blank_label, big_blank_durations, fastemit_lambda, clamp,
    num_threads=0, sigma=0.0, *, riders=None,
):  # fmt: skip
    """Multi-blank counterpart (rnnt.py:366-483): acts [B,T,U,V] with the big blanks at blank_label-1-i;
    costs is float32 [B], grads (or None) has the shape and dtype of acts."""
    del num_threads
    _require_gpu(acts, "multiblank_rnnt_loss_gpu")
    B, T, U, V = acts.shape
    workspace = new_workspace(acts, len(big_blank_durations))
    if costs.dtype != torch.float32:
        raise TypeError("costs must be float32")
    keep, dur_ptr = _durations_array(big_blank_durations)
    with torch.cuda.device(acts.device):
        status = _native.lib().mi_multiblank_loss(
            _ptr(acts), _dtype_code(acts), _labels_ptr(labels), _ptr(input_lengths), _ptr(label_lengths), _ptr(costs),
            _ptr(grads), None, 0, 1.0, B, T, U, V, len(big_blank_durations), dur_ptr, int(blank_label),
            float(fastemit_lambda), float(clamp), float(sigma), _riders_code(riders), _ptr(workspace),
            workspace.numel(), _stream(acts.device),
        )  # fmt: skip
    del keep
    _native.check_status(status, "Could not calculate forward scores")
    return True
