from .train import LogprobsPostProcessor

__all__ = ["LogprobsPostProcessor"]
