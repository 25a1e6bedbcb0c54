"""Ops that serve the graph-based (k2) transducer losses: the compact log-prob op."""

from speech_amd.k2.rnnt_logprobs import RnntLogProbs, rnnt_logprobs, rnnt_logprobs_triton

__all__ = ["RnntLogProbs", "rnnt_logprobs", "rnnt_logprobs_triton"]
