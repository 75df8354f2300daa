"""Alias of :mod:`rl_amd.algorithms.loss.loss_functions` under the shorter dotted path."""

from .loss.loss_functions import *  # noqa: F401,F403
from .loss.loss_functions import ClippedPGLossConfig, ClippedPGLossFn, NLLLossFn  # noqa: F401
