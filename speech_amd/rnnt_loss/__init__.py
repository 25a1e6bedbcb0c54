from speech_amd.rnnt_loss.rnnt import rnnt_loss_gpu, tdt_loss_gpu
from speech_amd.rnnt_loss.rnnt_pytorch import (
    RNNTLossMI355X,
    RNNTLossNumba,
    TDTLossMI355X,
    TDTLossNumba,
    certify_inputs,
)

__all__ = [
    'rnnt_loss_gpu',
    'tdt_loss_gpu',
    'RNNTLossNumba',
    'TDTLossNumba',
    'RNNTLossMI355X',
    'TDTLossMI355X',
    'certify_inputs',
]
