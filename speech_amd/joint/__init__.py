"""Joint projection fused into the transducer loss (the [B,T,U,V] tensor is never written)."""

from speech_amd.joint.fused import joint_rnnt_forward

__all__ = ["joint_rnnt_forward"]
