"""GRPO loss, sampling filter and advantage estimation (counterparts of ``nemo_rl.algorithms``)."""
