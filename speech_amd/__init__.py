"""MI355X-native transducer loss (RNNT / TDT / multi-blank) behind NeMo's *LossNumba call surface."""

from speech_amd.rnnt_loss import (  # noqa: F401
    MultiblankRNNTLossMI355X,
    MultiblankRNNTLossNumba,
    RNNTLossMI355X,
    RNNTLossNumba,
    TDTLossMI355X,
    TDTLossNumba,
    certify_inputs,
    multiblank_rnnt_loss_gpu,
    rnnt_loss_gpu,
    tdt_loss_gpu,
)

__version__ = "0.1.0"
