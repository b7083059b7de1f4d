from .fire import FIRE

__all__ = ["FIRE"]
