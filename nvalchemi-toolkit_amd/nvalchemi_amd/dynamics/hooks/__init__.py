from ._utils import (KB_EV, kinetic_energy_per_graph, scatter_reduce_per_graph, temperature_per_graph)

__all__ = ["KB_EV", "kinetic_energy_per_graph", "scatter_reduce_per_graph", "temperature_per_graph"]
