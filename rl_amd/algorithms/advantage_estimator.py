"""GRPO advantage estimator (counterpart of ``nemo_rl/algorithms/advantage_estimator.py:44-98``)."""

from __future__ import annotations

import torch
from pydantic import BaseModel

from .utils import _group_stats, _host_only


class AdvEstimatorConfig(BaseModel, extra="allow"):
    """``advantage_estimator.py:44-54``."""

    name: str = "grpo"
    normalize_rewards: bool = True
    use_leave_one_out_baseline: bool = True
    reward_weights: list[float] | None = None
    minus_baseline: bool = True


class GRPOAdvantageEstimator:
    """Leave-one-out (or full) group baseline, optional division by the group std."""

    def __init__(self, estimator_config, loss_config):
        self.use_leave_one_out_baseline = estimator_config.use_leave_one_out_baseline
        self.normalize_rewards = estimator_config.normalize_rewards
        self._configs = (estimator_config, loss_config)

    def compute_advantage(self, prompt_ids, rewards, mask, **kwargs):
        """``advantage_estimator.py:82-98``: ``[B]`` rewards -> ``[B, S]`` advantages (a stride-0
        expansion along the sequence, like the reference).  Grouping, statistics, the subtraction and
        the ``std > 0`` normalisation by ``std + 1e-6`` run in one HIP call.  On a NeMo-RL install, host
        tensors in a process that sees no GPU (a driver on a CPU node) go to the class the install came with."""
        if _host_only(prompt_ids, rewards, mask):
            from ..compat import original

            theirs = original("nemo_rl.algorithms.advantage_estimator", "GRPOAdvantageEstimator")
            if theirs is not None:
                return theirs(*self._configs).compute_advantage(prompt_ids, rewards, mask, **kwargs)
        _, _, adv, _ = _group_stats(
            prompt_ids, rewards, torch.ones_like(rewards), self.use_leave_one_out_baseline, None,
            self.normalize_rewards,
        )
        return adv.unsqueeze(-1).expand(mask.shape)
