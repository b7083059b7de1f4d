from .fire import FIRE
from .fire2 import FIRE2

__all__ = ["FIRE", "FIRE2"]
