"""MI355X-native batched MD inner loop behind the nvalchemi interfaces for that path.

Sub-modules mirror the reference layout: ``neighbors`` (``compute_neighbors``),
``hooks`` (``NeighborListHook``), ``models`` (``LennardJonesModelWrapper``), ``dynamics``
(``BaseDynamics``, ``NVE``, ``FIRE``), ``data`` (``Batch``, ``AtomicData``).  The kernels
live in ``lib/libnvalchemi_amd.so`` and are reached through ``_lib`` (ctypes over a C ABI).
"""

__version__ = "0.1.0"
