from .base import BaseModelMixin, ModelConfig, NeighborConfig, NeighborListFormat

__all__ = ["BaseModelMixin", "ModelConfig", "NeighborConfig", "NeighborListFormat",
           "LennardJonesModelWrapper"]


def __getattr__(name):
    if name == "LennardJonesModelWrapper":
        from .lj import LennardJonesModelWrapper

        return LennardJonesModelWrapper
    raise AttributeError(name)
