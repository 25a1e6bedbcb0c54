"""Module-level call surface of the transducer loss on MI355X.

Keeps the interface of nemo/collections/asr/parts/numba/rnnt_loss/rnnt_pytorch.py:
`RNNTLossNumba` (:392-439) and `TDTLossNumba` (:513-583) with the same
constructor arguments, the same `forward(acts, labels, act_lens, label_lens)`
(names and order are part of the contract: the outer wrapper calls by keyword,
nemo/collections/asr/losses/rnnt.py:484-491), the same mutable attributes
(`blank`, `reduction`, `fastemit_lambda`, `clamp`, `durations`, `sigma`, `omega`),
the same input validation and exceptions (`certify_inputs`, :601-634) and the
same outputs: float32 costs of shape [B] (reduction None/'none') or [1]
('sum'/'mean'), gradient only w.r.t. `acts`.

What is done differently underneath:
  * `acts` are raw logits of dtype float32, bfloat16 or float16 on the GPU; the
    log-softmax happens inside the kernels.  CPU tensors go to the host library (RNNT
    only, as in the reference; TDT and multi-blank raise there as they do in the reference).
  * the gradient is computed in `backward`, by one kernel pass that already folds
    in `grad_output`, the 'mean' reduction's 1/B, FastEmit and the clamp.  For logits
    below 32 MiB forward keeps only a few MB of lattice state; from 32 MiB on (and when
    acts requires a gradient) forward ALSO allocates the gradient tensor, the size of
    `acts`, as the reference does (which computes the gradient there): the lattice launch
    zero-fills its padded cells while it runs.  That tensor is held until backward runs or
    the graph is dropped; MI_TRANSDUCER_PREFILL=0 in the environment restores the small footprint.
  * the shape-vs-lengths check reads both maxima back with one small copy that
    overlaps the forward kernels instead of two blocking torch.max calls.
"""

import contextlib
import os
import random
import threading
import weakref

import torch
from torch.autograd import Function
from torch.nn import Module

from speech_amd.rnnt_loss import rnnt

__all__ = [
    'RNNTLossNumba', 'TDTLossNumba', 'MultiblankRNNTLossNumba', 'RNNTLossMI355X', 'TDTLossMI355X',
    'MultiblankRNNTLossMI355X', 'certify_inputs',
]  # fmt: skip



# The gradient of padded cells is zeros that depend on the lengths alone.  When the gradient will be needed, forward
# allocates it and hands it to the lattice launch, whose extra workgroups write those zeros while the recursion runs
# and HBM would idle (rnnt.rnnt_forward, prefill_grads); backward then skips what they did.  Measured fwd+bwd at B=16,
# T=375, U=121, V=1025 fp32: RNNT 1.146 -> 1.124 ms, TDT 1.35 -> 1.185 ms, multi-blank 1.27 -> 1.16 ms.
# MI_TRANSDUCER_PREFILL=0 switches it off.
_PREFILL_ENV = os.environ.get("MI_TRANSDUCER_PREFILL", "")
_PREFILL_MIN_BYTES = 32 << 20  # below this a step is bound by its launches


def _prefill_wanted(acts):
    if _PREFILL_ENV in ("0", "1"):
        return _PREFILL_ENV == "1"
    return acts.numel() * acts.element_size() >= _PREFILL_MIN_BYTES


_aux_streams = {}


def _aux_stream(device):
    stream = _aux_streams.get(device.index)
    if stream is None:
        stream = torch.cuda.Stream(device=device)  # default priority
        _aux_streams[device.index] = stream
    return stream


def grads_like(acts):
    """An uninitialised tensor of the shape and dtype of acts whose storage starts at the same offset within a
    256-byte block as acts does.  The gradient pass stores whole 16-byte vectors where the logits row has them, which
    needs the two buffers in phase, and its stores stream when each instruction covers whole 64-byte pieces, which
    they do when the phases agree that far; a fresh allocation is 256-byte aligned, a view such as `big[1:]` need
    not be."""
    phase = acts.data_ptr() & 255
    if phase == 0:
        return torch.empty_like(acts)
    size = acts.element_size()
    flat = torch.empty(acts.numel() + 256 // size, dtype=acts.dtype, device=acts.device)
    first = ((phase - flat.data_ptr()) & 255) // size
    return flat[first : first + acts.numel()].view(acts.shape)


def check_type(var, t, name):
    if var.dtype is not t:
        raise TypeError("{} must be {}".format(name, t))


def check_contiguous(var, name):
    if not var.is_contiguous():
        raise ValueError("{} must be contiguous".format(name))


def check_dim(var, dim, name):
    if len(var.shape) != dim:
        raise ValueError("{} must be {}D".format(name, dim))


class _CallerMode(threading.local):
    """How the next module call treats two things a wrapper around it decides (set only by
    speech_amd.losses.rnnt.RNNTLoss, which stands where nemo/collections/asr/losses/rnnt.py:438-505 stands):
    padded_time_axis  accept T >= max(act_lens): the wrapper of the reference trims the time axis with
                      narrow().contiguous() before the call; the kernels skip padded frames anyway, so
                      the copy is not made and the frames beyond max(act_lens) get a zero gradient
    float32_costs     keep the costs in float32 whatever the dtype of acts (the reference's wrapper
                      upcasts 16-bit logits before the call, so its costs are float32)"""

    padded_time_axis = False
    float32_costs = False


_caller_mode = _CallerMode()


@contextlib.contextmanager
def wrapper_call_mode():
    old = (_caller_mode.padded_time_axis, _caller_mode.float32_costs)
    _caller_mode.padded_time_axis = _caller_mode.float32_costs = True
    try:
        yield
    finally:
        _caller_mode.padded_time_axis, _caller_mode.float32_costs = old


class _ValidatedLengths(threading.local):
    """The last pair of length tensors that passed the shape check on this thread: (weak reference, version) of each
    and the shape they were checked against.  Calling again with the SAME tensor objects, unmodified (torch bumps a
    tensor's version on every in-place write), against the same shape cannot give another answer, so the read-back
    and the host wait it costs are skipped -- repeated calls on one batch (gradient accumulation, benchmarks) then
    never block the host.  Writes that bypass the version counter (`.data`, foreign kernels) are not seen; what is
    lost then is only the ValueError for a malformed batch, the kernels clamp lengths anyway.
    MI_TRANSDUCER_STRICT_LENGTH_CHECK=1 in the environment switches the memory off: every call then reads the maxima
    back, as certify_inputs of the reference does (rnnt_pytorch.py:628-634)."""

    entry = None


_validated = _ValidatedLengths()
_STRICT_LENGTH_CHECK = os.environ.get("MI_TRANSDUCER_STRICT_LENGTH_CHECK", "") == "1"


class _PendingLengthCheck:
    """The T == max(act_lens), U == max(label_lens)+1 test of certify_inputs, split in two
    so that the read-back of the maxima overlaps kernels enqueued in between."""

    def __init__(self, log_probs, lengths, label_lengths):
        self.T, self.U = log_probs.shape[1:3]
        self.padded_T = _caller_mode.padded_time_axis
        self.key = (lengths._version, label_lengths._version, self.T, self.U, self.padded_T)
        self.tensors = (lengths, label_lengths)
        self.event = self.host = None
        seen = _validated.entry
        if (not _STRICT_LENGTH_CHECK and seen is not None and seen[0]() is lengths and seen[1]() is label_lengths
                and seen[2] == self.key):
            return  # these very tensors, unmodified, passed against this shape
        if lengths.is_cuda:
            # One small kernel on the auxiliary stream, ordered after whatever produced the lengths
            # on the current stream, writes the two maxima into pinned host memory: it runs beside
            # the first kernel of the loss instead of in front of it.
            main = torch.cuda.current_stream(lengths.device)
            aux = _aux_stream(lengths.device)
            aux.wait_stream(main)
            self.host = torch.empty(2, dtype=torch.int64, pin_memory=True)
            with torch.cuda.stream(aux):
                rnnt.length_maxima(lengths, label_lengths, out=self.host)
                self.event = torch.cuda.Event()
                self.event.record(aux)
            lengths.record_stream(aux)
            label_lengths.record_stream(aux)
        else:
            self.host = torch.stack([torch.max(lengths), torch.max(label_lengths)])

    def drain(self):
        """Wait for the kernel that writes into the pinned buffer, so that the buffer is not handed back to the host
        allocator (and on to some other user) while that write is still queued.  For the error paths that drop
        this object without finish()."""
        if self.event is not None:
            self.event.synchronize()
            self.event = None

    def finish(self):
        if self.host is None:
            return
        self.drain()
        max_T, max_U = int(self.host[0]), int(self.host[1])
        if self.T < max_T if self.padded_T else self.T != max_T:
            raise ValueError(f"Input length mismatch! Given T: {self.T}, Expected max T from input lengths: {max_T}")
        if self.U != max_U + 1:
            raise ValueError(
                f"Output length mismatch! Given U: {self.U}, Expected max U from target lengths: {max_U} + 1"
            )
        lengths, label_lengths = self.tensors
        if (lengths._version, label_lengths._version) == self.key[:2]:
            _validated.entry = (weakref.ref(lengths), weakref.ref(label_lengths), self.key)


def _certify_static(log_probs, labels, lengths, label_lengths):
    check_type(labels, torch.int64, "labels")
    check_type(label_lengths, torch.int64, "label_lengths")
    check_type(lengths, torch.int64, "lengths")
    check_contiguous(log_probs, "log_probs")
    check_contiguous(labels, "labels")
    check_contiguous(label_lengths, "label_lengths")
    check_contiguous(lengths, "lengths")

    if lengths.shape[0] != log_probs.shape[0]:
        raise ValueError(
            f"Must have a length per example. "
            f"Given lengths dim: {lengths.shape[0]}, "
            f"Log probs dim : {log_probs.shape[0]}"
        )
    if label_lengths.shape[0] != log_probs.shape[0]:
        raise ValueError(
            "Must have a label length per example. "
            f"Given label lengths dim : {label_lengths.shape[0]}, "
            f"Log probs dim : {log_probs.shape[0]}"
        )

    check_dim(log_probs, 4, "log_probs")
    check_dim(labels, 2, "labels")
    check_dim(lengths, 1, "lenghts")
    check_dim(label_lengths, 1, "label_lenghts")


def certify_inputs(log_probs, labels, lengths, label_lengths):
    """Same checks, order, exception types and messages as rnnt_pytorch.py:601-634."""
    _certify_static(log_probs, labels, lengths, label_lengths)
    _PendingLengthCheck(log_probs, lengths, label_lengths).finish()


def _check_same_device(acts, *others):
    for t in others:
        if t.device != acts.device:
            raise ValueError(f"labels and lengths must be on the device of acts ({acts.device}), got {t.device}")


def _reduce_costs(costs, reduction, batch):
    # rnnt_pytorch.py:75-81: 'sum' and 'mean' give shape [1]; anything else is per utterance
    if reduction in ['sum', 'mean']:
        costs = costs.sum().unsqueeze_(-1)
        if reduction == 'mean':
            costs /= batch
    return costs


def _grad_scale(grad_output, reduction, batch, device):
    """(tensor, stride, multiplier) such that utterance b's gradient is scaled by
    tensor[b * stride] * multiplier: what the reference applies to its stored gradient -- 1/B for
    'mean' in forward (rnnt_pytorch.py:77-81), then grad_output broadcast over the batch in backward
    (:88-92).  The usual cases (a dense or a broadcast float32 grad_output) need no copy."""
    mul = 1.0 / batch if reduction == 'mean' else 1.0
    g = grad_output.detach()
    if g.dtype != torch.float32 or g.device != device:
        g = g.to(device=device, dtype=torch.float32)
    if g.numel() == 1:
        return g.reshape(1), 0, mul
    if g.numel() != batch:
        raise RuntimeError(f"grad_output has {g.numel()} elements, expected 1 or {batch}")
    if g.dim() != 1:
        g = g.reshape(batch)
    return g, g.stride(0), mul


class _RNNTNumba(Function):
    @staticmethod
    def forward(ctx, acts, labels, act_lens, label_lens, blank, reduction, fastemit_lambda, clamp):
        _certify_static(acts, labels, act_lens, label_lens)
        if clamp < 0:
            raise ValueError("`clamp` must be 0.0 or positive float value.")
        _check_same_device(acts, labels, act_lens, label_lens)
        ctx.on_cpu = not acts.is_cuda
        if ctx.on_cpu:
            # the host library (rnnt_pytorch.py:420-435 + cpu_utils/cpu_rnnt.py): float32 logits in, float32 costs out
            _PendingLengthCheck(acts, act_lens, label_lens).finish()
            if acts.dtype != torch.float32:
                raise TypeError("RNNTLossNumba on CPU tensors computes in float32: the module casts 16-bit logits")
            need_grad = ctx.needs_input_grad[0]
            batch = acts.size(0)
            costs = torch.empty(batch, dtype=torch.float32)
            workspace = rnnt.cpu_workspace(acts)
            rnnt.rnnt_cpu_forward(acts, labels, act_lens, label_lens, costs, blank, fastemit_lambda, workspace)
            costs = _reduce_costs(costs, reduction, batch)
            if need_grad:
                ctx.save_for_backward(acts, labels, act_lens, label_lens, workspace)
                ctx.params = (blank, reduction, fastemit_lambda, clamp)
            return costs
        pending = _PendingLengthCheck(acts, act_lens, label_lens)
        try:
            need_grad = ctx.needs_input_grad[0]
            batch = acts.size(0)
            costs = torch.empty(batch, device=acts.device, dtype=torch.float32)
            workspace = rnnt.new_workspace(acts)
            ctx.prefilled = grads_like(acts) if need_grad and _prefill_wanted(acts) else None
            rnnt.rnnt_forward(acts, labels, act_lens, label_lens, costs, blank, fastemit_lambda, need_grad, workspace,
                              ctx.prefilled)
        except BaseException:
            pending.drain()  # the pinned buffer must outlive the kernel that writes into it
            raise
        pending.finish()  # raises ValueError exactly where certify_inputs would

        costs = _reduce_costs(costs, reduction, batch)
        if need_grad:
            ctx.save_for_backward(acts, labels, act_lens, label_lens, workspace)
            ctx.params = (blank, reduction, fastemit_lambda, clamp)
        return costs

    @staticmethod
    def backward(ctx, grad_output):
        acts, labels, act_lens, label_lens, workspace = ctx.saved_tensors
        blank, reduction, fastemit_lambda, clamp = ctx.params
        if ctx.on_cpu:
            grads = torch.empty_like(acts)
            scale, stride, mul = _grad_scale(grad_output, reduction, acts.size(0), acts.device)
            scale = scale.contiguous()  # (a broadcast grad_output is materialised: B floats)
            rnnt.rnnt_cpu_backward(acts, labels, act_lens, label_lens, grads, scale, blank, fastemit_lambda, clamp,
                                   workspace, 1 if scale.numel() > 1 else 0, mul)  # fmt: skip
            return grads, None, None, None, None, None, None, None
        prefilled, ctx.prefilled = ctx.prefilled, None  # the prefilled buffer serves the first backward call only
        grads = prefilled if prefilled is not None else grads_like(acts)
        scale, stride, mul = _grad_scale(grad_output, reduction, acts.size(0), acts.device)
        rnnt.rnnt_backward(
            acts, labels, act_lens, label_lens, grads, scale, blank, fastemit_lambda, clamp, workspace, stride, mul,
            2 if prefilled is not None else 0,
        )  # fmt: skip
        return grads, None, None, None, None, None, None, None


class _TDTNumba(Function):
    """Token-and-Duration Transducer loss (arXiv:2304.06795) on the combined logits."""

    @staticmethod
    def forward(
        ctx, acts, labels, act_lens, label_lens, blank, durations, reduction, fastemit_lambda, clamp, sigma, omega
    ):
        _certify_static(acts, labels, act_lens, label_lens)
        if clamp < 0:
            raise ValueError("`clamp` must be 0.0 or positive float value.")
        if not acts.is_cuda:
            # rnnt_pytorch.py:137-140
            raise ValueError("TDT is not yet implemented for non CUDA computation.")
        _check_same_device(acts, labels, act_lens, label_lens)
        durations = [int(d) for d in durations]
        if acts.shape[-1] <= len(durations):
            raise ValueError("acts must hold the token logits followed by one logit per duration")
        pending = _PendingLengthCheck(acts, act_lens, label_lens)
        try:
            need_grad = ctx.needs_input_grad[0]
            batch = acts.size(0)
            costs = torch.empty(batch, device=acts.device, dtype=torch.float32)
            workspace = rnnt.new_workspace(acts, len(durations))
            # gpu_rnnt.py:606-607: one host-side draw per call decides between the TDT and the plain RNNT kernels
            use_plain_rnnt = random.uniform(0, 1) < omega
            ctx.prefilled = grads_like(acts) if need_grad and _prefill_wanted(acts) else None
            rnnt.tdt_forward(
                acts, labels, act_lens, label_lens, costs, blank, durations, fastemit_lambda, sigma, use_plain_rnnt,
                need_grad, workspace, ctx.prefilled,
            )  # fmt: skip
        except BaseException:
            pending.drain()  # the pinned buffer must outlive the kernel that writes into it
            raise
        pending.finish()

        # the reference allocates TDT costs in the dtype of acts (rnnt_pytorch.py:145)
        costs = _reduce_costs(costs, reduction, batch)
        if not _caller_mode.float32_costs:
            costs = costs.to(acts.dtype)
        if need_grad:
            ctx.save_for_backward(acts, labels, act_lens, label_lens, workspace)
            ctx.params = (blank, durations, reduction, fastemit_lambda, clamp, sigma, use_plain_rnnt)
        return costs

    @staticmethod
    def backward(ctx, grad_output):
        acts, labels, act_lens, label_lens, workspace = ctx.saved_tensors
        blank, durations, reduction, fastemit_lambda, clamp, sigma, use_plain_rnnt = ctx.params
        prefilled, ctx.prefilled = ctx.prefilled, None  # (serves the first backward call only)
        grads = prefilled if prefilled is not None else grads_like(acts)
        scale, stride, mul = _grad_scale(grad_output, reduction, acts.size(0), acts.device)
        rnnt.tdt_backward(
            acts, labels, act_lens, label_lens, grads, scale, blank, durations, fastemit_lambda, clamp, sigma,
            use_plain_rnnt, workspace, stride, mul, 2 if prefilled is not None else 0,
        )  # fmt: skip
        return grads, None, None, None, None, None, None, None, None, None, None


class _MultiblankRNNTNumba(Function):
    """Multi-blank transducer loss (arXiv:2211.03541); rnnt_pytorch.py:199-268."""

    @staticmethod
    def forward(
        ctx, acts, labels, act_lens, label_lens, blank, big_blank_durations, reduction, fastemit_lambda, clamp, sigma
    ):
        _certify_static(acts, labels, act_lens, label_lens)
        if clamp < 0:
            raise ValueError("`clamp` must be 0.0 or positive float value.")
        if not acts.is_cuda:
            raise NotImplementedError()  # rnnt_pytorch.py:226-229
        _check_same_device(acts, labels, act_lens, label_lens)
        durations = [int(d) for d in big_blank_durations]
        if blank - len(durations) < 0 or blank >= acts.shape[-1]:
            raise ValueError("the big blanks sit at blank-1-i: blank must leave room for them below it")
        pending = _PendingLengthCheck(acts, act_lens, label_lens)
        try:
            need_grad = ctx.needs_input_grad[0]
            batch = acts.size(0)
            costs = torch.empty(batch, device=acts.device, dtype=torch.float32)
            workspace = rnnt.new_workspace(acts, len(durations))
            ctx.prefilled = grads_like(acts) if need_grad and _prefill_wanted(acts) else None
            rnnt.multiblank_forward(
                acts, labels, act_lens, label_lens, costs, blank, durations, fastemit_lambda, sigma, need_grad, workspace,
                ctx.prefilled,
            )  # fmt: skip
        except BaseException:
            pending.drain()  # the pinned buffer must outlive the kernel that writes into it
            raise
        pending.finish()

        # the reference allocates these costs in the dtype of acts (rnnt_pytorch.py:232)
        costs = _reduce_costs(costs, reduction, batch)
        if not _caller_mode.float32_costs:
            costs = costs.to(acts.dtype)
        if need_grad:
            ctx.save_for_backward(acts, labels, act_lens, label_lens, workspace)
            ctx.params = (blank, durations, reduction, fastemit_lambda, clamp, sigma)
        return costs

    @staticmethod
    def backward(ctx, grad_output):
        acts, labels, act_lens, label_lens, workspace = ctx.saved_tensors
        blank, durations, reduction, fastemit_lambda, clamp, sigma = ctx.params
        prefilled, ctx.prefilled = ctx.prefilled, None  # (serves the first backward call only)
        grads = prefilled if prefilled is not None else grads_like(acts)
        scale, stride, mul = _grad_scale(grad_output, reduction, acts.size(0), acts.device)
        rnnt.multiblank_backward(
            acts, labels, act_lens, label_lens, grads, scale, blank, durations, fastemit_lambda, clamp, sigma,
            workspace, stride, mul, 2 if prefilled is not None else 0,
        )  # fmt: skip
        return grads, None, None, None, None, None, None, None, None, None


class RNNTLossNumba(Module):
    """
    Parameters:
        blank (int, optional): blank label. Default: 0.
        reduction (string, optional): 'none' | 'mean' | 'sum' (None behaves as 'none'). Default: 'mean'
        fastemit_lambda: scaling factor of the FastEmit regularisation (arXiv:2010.11148).
        clamp: when > 0, every gradient element is clamped to [-clamp, clamp]; <= 0 disables it.
    """

    def __init__(self, blank=0, reduction='mean', fastemit_lambda: float = 0.0, clamp: float = -1):
        super().__init__()
        self.blank = blank
        self.fastemit_lambda = fastemit_lambda
        self.clamp = float(clamp) if clamp > 0 else 0.0
        self.reduction = reduction
        self.loss = _RNNTNumba.apply

    def forward(self, acts, labels, act_lens, label_lens):
        """
        acts: [B, T, U, V] logits from the joint network (blank included in V)
        labels: [B, U-1] int64 targets, zero padded
        act_lens: [B] int64 number of valid frames per utterance
        label_lens: [B] int64 number of valid labels per utterance
        """
        if not acts.is_cuda and acts.dtype != torch.float32:
            # rnnt_pytorch.py:422-424: 16-bit logits are computed in float32 on the CPU; autograd casts the gradient back
            acts = acts.float()
        return self.loss(
            acts, labels, act_lens, label_lens, self.blank, self.reduction, self.fastemit_lambda, self.clamp
        )


class TDTLossNumba(Module):
    """
    Parameters:
        blank (int): blank label (index within the token logits).
        durations: durations of the TDT model, ascending, e.g. [0, 1, 2, 3, 4]; must hold 1 at position 0 or 1.
        reduction, fastemit_lambda, clamp: as RNNTLossNumba.
        sigma: logit under-normalisation constant (recommended 0.05).
        omega: probability of using the plain RNNT loss for a call.
    """

    def __init__(
        self,
        blank,
        durations=None,
        reduction='mean',
        fastemit_lambda: float = 0.0,
        clamp: float = -1,
        sigma: float = 0.0,
        omega: float = 0.0,
    ):
        super().__init__()
        self.blank = blank
        self.durations = durations if durations is not None else []
        self.fastemit_lambda = fastemit_lambda
        self.clamp = float(clamp) if clamp > 0 else 0.0
        self.reduction = reduction
        self.loss = _TDTNumba.apply
        self.sigma = sigma
        self.omega = omega

    def forward(self, acts, labels, act_lens, label_lens):
        """
        acts: [B, T, U, V + D] logits: V token logits (blank included) then D = len(durations) duration logits
        labels, act_lens, label_lens: as RNNTLossNumba
        """
        return self.loss(
            acts,
            labels,
            act_lens,
            label_lens,
            self.blank,
            self.durations,
            self.reduction,
            self.fastemit_lambda,
            self.clamp,
            self.sigma,
            self.omega,
        )


class MultiblankRNNTLossNumba(Module):
    """
    Parameters:
        blank (int): standard blank label.
        big_blank_durations: durations of the big blanks, e.g. [2, 4, 8]; big blank i is token blank-1-i.
        reduction, fastemit_lambda, clamp: as RNNTLossNumba.
        sigma: logit under-normalisation constant (recommended 0.05).
    """

    def __init__(
        self,
        blank,
        big_blank_durations,
        reduction='mean',
        fastemit_lambda: float = 0.0,
        clamp: float = -1,
        sigma: float = 0.0,
    ):
        super().__init__()
        self.blank = blank
        self.big_blank_durations = big_blank_durations
        self.fastemit_lambda = fastemit_lambda
        self.clamp = float(clamp) if clamp > 0 else 0.0
        self.reduction = reduction
        self.loss = _MultiblankRNNTNumba.apply
        self.sigma = sigma

    def forward(self, acts, labels, act_lens, label_lens):
        """
        acts: [B, T, U, V] logits over the tokens, the big blanks and the standard blank
        labels, act_lens, label_lens: as RNNTLossNumba
        """
        return self.loss(
            acts,
            labels,
            act_lens,
            label_lens,
            self.blank,
            self.big_blank_durations,
            self.reduction,
            self.fastemit_lambda,
            self.clamp,
            self.sigma,
        )


# names that say what they are; the *Numba names are kept so that code written
# against the reference runs unchanged
RNNTLossMI355X = RNNTLossNumba
TDTLossMI355X = TDTLossNumba
MultiblankRNNTLossMI355X = MultiblankRNNTLossNumba
