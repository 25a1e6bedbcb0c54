"""The loss wrapper a transducer model constructs: name resolution, casting, reduction.

Mirrors nemo/collections/asr/losses/rnnt.py: `RNNTLossConfig` / `RNNT_LOSS_RESOLVER` (:77-158),
`resolve_rnnt_loss` (:206-330) and `RNNTLoss` (:333-505) with the same constructor, the same
keyword-only `forward(log_probs=, targets=, input_lengths=, target_lengths=)`, the same reductions
(`mean_batch`, `mean`, `sum`, `mean_volume`, None) and the same exceptions.  The names this build
implements are "warprnnt_numba" (= "default"), "tdt" and "multiblank_rnnt"; the others stay in the
table, marked unavailable, so that selecting one fails the way an uninstalled backend fails there.

What is done differently underneath:
  * nothing is upcast: 16-bit joint tensors are read as they are (the kernels accumulate in
    fp32/fp64 and round the gradient once), where the reference converts the whole tensor to fp32
    first (:449-465).  Costs stay float32 either way.
  * nothing is trimmed: when the time axis is longer than max(input_lengths) the reference copies the
    tensor (`narrow().contiguous()`, :473-474, after a host sync on the maximum) and autograd later
    pads the gradient back; here the full tensor goes to the kernels, which skip padded frames and
    zero-fill their gradient.  Only the (tiny) target matrix is trimmed when it is wider than needed.
"""

import logging
from dataclasses import dataclass
from typing import List, Optional

import torch

from speech_amd.rnnt_loss import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba
from speech_amd.rnnt_loss.rnnt_pytorch import wrapper_call_mode

__all__ = ['RNNTLoss', 'RNNTLossConfig', 'RNNT_LOSS_RESOLVER', 'resolve_rnnt_loss', 'resolve_rnnt_default_loss_name']

_NATIVE_MESSAGE = "Built into this package (HIP kernels for MI355X); nothing to install."
_ABSENT_MESSAGE = (
    "This loss is not part of the MI355X build, which implements `warprnnt_numba`, `tdt` and `multiblank_rnnt`."
)


@dataclass
class RNNTLossConfig:
    loss_name: str
    lib_name: str
    is_available: bool = False
    installation_msg: str = ""
    min_version: Optional[str] = None
    force_float32: bool = True


def _native(name):
    # force_float32 False: 16-bit logits are consumed natively (see the module docstring)
    return RNNTLossConfig(loss_name=name, lib_name="speech_amd", is_available=True,
                          installation_msg=_NATIVE_MESSAGE, force_float32=False)  # fmt: skip


def _absent(name, lib):
    return RNNTLossConfig(loss_name=name, lib_name=lib, is_available=False, installation_msg=_ABSENT_MESSAGE)


# the names of nemo/collections/asr/losses/rnnt.py:88-156
RNNT_LOSS_RESOLVER = {
    "warprnnt": _absent("warprnnt", "warprnnt_pytorch"),
    "warprnnt_numba": _native("warprnnt_numba"),
    "pytorch": _absent("pytorch", "torch"),
    "multiblank_rnnt": _native("multiblank_rnnt"),
    "multiblank_rnnt_pytorch": _absent("pytorch", "torch"),
    "graph_w_transducer": _absent("graph_w_transducer", "k2"),
    "graph_rnnt": _absent("graph_rnnt", "k2"),
    "tdt": _native("tdt"),
    "tdt_pytorch": _absent("tdt_pytorch", "torch"),
}
RNNT_LOSS_RESOLVER['default'] = RNNT_LOSS_RESOLVER['warprnnt_numba']


def _listed(value, empty):
    return list(value) if value is not None else empty


# name -> (module class, keyword defaults in the order the reference pops them (losses/rnnt.py:264-310), and what
# to do with a value on its way into the constructor).  Keyword names and defaults are the reference's contract.
_CONSTRUCTORS = {
    'warprnnt_numba': (RNNTLossNumba, {'fastemit_lambda': 0.0, 'clamp': -1.0}, {}),
    'multiblank_rnnt': (
        MultiblankRNNTLossNumba,
        {'fastemit_lambda': 0.0, 'clamp': -1.0, 'big_blank_durations': None, 'sigma': 0.0},
        {'big_blank_durations': lambda v: _listed(v, [])},
    ),
    'tdt': (
        TDTLossNumba,
        {'fastemit_lambda': 0.0, 'clamp': -1.0, 'durations': None, 'sigma': 0.0, 'omega': 0.0},
        {'durations': lambda v: _listed(v, None)},
    ),
}


def resolve_rnnt_default_loss_name() -> str:
    return RNNT_LOSS_RESOLVER['default'].loss_name


def resolve_rnnt_loss(loss_name: str, blank_idx: int, loss_kwargs: dict = None) -> torch.nn.Module:
    """losses/rnnt.py:206-330: the loss module for `loss_name`, always built with reduction='none'."""
    loss_function_names = list(RNNT_LOSS_RESOLVER.keys())
    if loss_name not in loss_function_names:
        raise ValueError(
            f"Provided `loss_name` {loss_name} not in list of available RNNT losses \n" f"{loss_function_names}"
        )
    all_available_losses = {name: config for name, config in RNNT_LOSS_RESOLVER.items() if config.is_available}
    loss_config = RNNT_LOSS_RESOLVER[loss_name]
    if not loss_config.is_available:
        raise ImportError(
            f"Installed RNNT losses are : {list(all_available_losses.keys())}.\n"
            f"****************************************************************\n"
            f"To install the selected loss function, please follow the steps below:\n"
            f"{loss_config.installation_msg}"
        )
    # a mapping from a config system (e.g. an OmegaConf DictConfig) is taken as a plain dict; it is copied
    # because the known arguments are popped from it
    loss_kwargs = {} if loss_kwargs is None else {k: loss_kwargs[k] for k in loss_kwargs}
    if loss_name == 'default':
        loss_name = loss_config.loss_name

    if loss_name not in _CONSTRUCTORS:  # an available name without a constructor: the two tables disagree
        raise ValueError(
            f"Invalid value of `loss_name`: {loss_name}. Allowed loss names are :" f"{loss_function_names}"
        )
    module_class, defaults, conversions = _CONSTRUCTORS[loss_name]
    arguments = {key: loss_kwargs.pop(key, default) for key, default in defaults.items()}
    for key, convert in conversions.items():
        arguments[key] = convert(arguments[key])
    loss_func = module_class(blank=blank_idx, reduction='none', **arguments)
    if loss_kwargs:  # whatever is left was not understood (losses/rnnt.py:161-167)
        logging.warning(
            f"Loss function `{loss_name}` was provided with following additional kwargs,\n"
            f"however they were ignored as it is unused.\n"
            f"{loss_kwargs}"
        )
    return loss_func


# reduction name -> (per-utterance losses [B], target lengths [B]) -> scalar (losses/rnnt.py:421-436)
_REDUCTIONS = {
    'mean_batch': lambda losses, lengths: losses.mean(),
    'mean': lambda losses, lengths: torch.div(losses, lengths).mean(),
    'sum': lambda losses, lengths: losses.sum(),
    'mean_volume': lambda losses, lengths: losses.sum() / lengths.sum(),
}


class RNNTLoss(torch.nn.Module):
    """losses/rnnt.py:333-505.  `num_classes` is the id of the standard blank: V for RNNT and TDT (the
    duration logits come after it), V + number of big blanks for the multi-blank loss."""

    def __init__(self, num_classes, reduction: str = 'mean_batch', loss_name: str = "default", loss_kwargs=None):
        super().__init__()
        if reduction is not None and reduction not in _REDUCTIONS:
            raise ValueError('`reduction` must be one of [mean, sum, mean_batch, mean_volume]')
        self._blank = num_classes
        self.reduction = reduction
        self._loss = resolve_rnnt_loss(loss_name, blank_idx=self._blank, loss_kwargs=loss_kwargs)
        self._force_float32 = RNNT_LOSS_RESOLVER[loss_name].force_float32

    def reduce(self, losses, target_lengths):
        if isinstance(losses, List):  # the fused joint hands over one tensor per sub-batch
            losses, target_lengths = torch.cat(losses, 0), torch.cat(target_lengths, 0)
        combine = _REDUCTIONS.get(self.reduction)
        return losses if combine is None else combine(losses, target_lengths)

    def forward(self, *args, log_probs=None, targets=None, input_lengths=None, target_lengths=None):
        if len(args) > 0:  # the reference's @typecheck() (nemo/core/classes/common.py:1357-1359)
            raise TypeError("All arguments must be passed by kwargs only for typed methods")
        targets = targets.long()
        input_lengths = input_lengths.long()
        target_lengths = target_lengths.long()
        if self._force_float32 and log_probs.dtype != torch.float32:
            log_probs = log_probs.float()  # only if a caller flips the flag back (losses/rnnt.py:449-465)
        if not log_probs.is_contiguous():
            log_probs = log_probs.contiguous()
        # Transcript: [B, L] -> [B, U-1] if extra padding was applied (losses/rnnt.py:478-481); the joint's
        # label axis says how long it has to be, which saves the reference's host sync on the maximum
        if targets.shape[1] > log_probs.shape[2] - 1:
            targets = targets.narrow(dim=1, start=0, length=log_probs.shape[2] - 1)
        if not targets.is_contiguous():
            targets = targets.contiguous()

        # Temporarily override loss reduction (losses/rnnt.py:484-491)
        loss_reduction = self._loss.reduction
        self._loss.reduction = None
        try:
            with wrapper_call_mode():
                loss = self._loss(acts=log_probs, labels=targets, act_lens=input_lengths, label_lens=target_lengths)
        finally:
            self._loss.reduction = loss_reduction

        if self.reduction is not None:
            loss = self.reduce(loss, target_lengths)
        return loss
