"""MI355X-native transducer loss (RNNT / TDT) behind NeMo's RNNTLossNumba / TDTLossNumba call surface."""

from speech_amd.rnnt_loss import (  # noqa: F401
    RNNTLossMI355X,
    RNNTLossNumba,
    TDTLossMI355X,
    TDTLossNumba,
    certify_inputs,
    rnnt_loss_gpu,
    tdt_loss_gpu,
)

__version__ = "0.1.0"
