"""Joint projection fused into the transducer loss (the [B,T,U,V] tensor is never written)."""

from speech_amd.joint.fused import (
    JointRNNTLoss,
    joint_dropout_mask,
    joint_multiblank_forward,
    joint_multiblank_loss,
    joint_rnnt_forward,
    joint_rnnt_loss,
    joint_tdt_forward,
    joint_tdt_loss,
)

__all__ = ["JointRNNTLoss", "joint_dropout_mask", "joint_multiblank_forward", "joint_multiblank_loss",
           "joint_rnnt_forward", "joint_rnnt_loss", "joint_tdt_forward", "joint_tdt_loss"]  # fmt: skip
