"""rl_amd: the GRPO training-side hot path (logits -> token logprobs -> clipped policy-gradient
loss, group advantages) as hand-written HIP kernels for MI355X (gfx950), behind the Python
signatures of NeMo-RL's ``nemo_rl.distributed.model_utils`` and ``nemo_rl.algorithms.*``.

``rl_amd.install()`` makes those dotted paths importable as ``nemo_rl.*`` (or patches an existing
NeMo-RL install) so a single-GPU policy worker picks the kernels up without code changes.
"""

__version__ = "0.1.0"

from .compat import install  # noqa: E402,F401
