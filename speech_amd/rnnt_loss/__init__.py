from speech_amd.rnnt_loss.rnnt import combined_tdt_loss_gpu, multiblank_rnnt_loss_gpu, rnnt_loss_gpu, tdt_loss_gpu
from speech_amd.rnnt_loss.rnnt_pytorch import (
    MultiblankRNNTLossMI355X,
    MultiblankRNNTLossNumba,
    RNNTLossMI355X,
    RNNTLossNumba,
    TDTLossMI355X,
    TDTLossNumba,
    certify_inputs,
)

__all__ = [
    'rnnt_loss_gpu',
    'tdt_loss_gpu',
    'combined_tdt_loss_gpu',
    'multiblank_rnnt_loss_gpu',
    'RNNTLossNumba',
    'TDTLossNumba',
    'MultiblankRNNTLossNumba',
    'RNNTLossMI355X',
    'TDTLossMI355X',
    'MultiblankRNNTLossMI355X',
    'certify_inputs',
]
