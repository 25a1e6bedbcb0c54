from speech_amd.losses.rnnt import (  # noqa: F401
    RNNT_LOSS_RESOLVER,
    RNNTLoss,
    RNNTLossConfig,
    resolve_rnnt_default_loss_name,
    resolve_rnnt_loss,
)
