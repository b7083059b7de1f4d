from .nve import NVE

__all__ = ["NVE"]
