"""Counterpart of ``nemo_rl/models/megatron``: the logprob post-processing of the Megatron worker."""

from .train import LogprobsPostProcessor

__all__ = ["LogprobsPostProcessor"]
