"""Writes the regression fixtures of this folder from the CPU oracle (never from the reference,
which cannot be imported here: its kernel library is absent).  Run from the repository root:

    python tests/golden/make_fixtures.py

`config1_molecules.npz`: BASELINE config 1 (seed 0; 8 molecules of 4..32 atoms, positions
N(0, 1.5 A), no cell; naive list at 5 A; LJ eps 0.01 eV, sigma 2.5 A; 100 velocity-Verlet steps of
0.5 fs from rest) -- the neighbor list and energies/forces of the start, and the state after the
trajectory.  `periodic_triclinic.npz`: four triclinic periodic boxes of 20..60 atoms with unwrapped
coordinates, list at 6 A -- neighbor rows with shifts, energies, forces, virials, 20 FIRE steps.

The fixtures pin the oracle against silent change (tests/test_golden_fixtures.py, CPU) and give
the GPU tests inputs and expected outputs that do not pass through the oracle at test time.
"""

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))
sys.path.insert(0, str(HERE.parent.parent))

import oracle  # noqa: E402
from _reference_loop import fire, nve  # noqa: E402
from _systems import molecules_batch, periodic_batch  # noqa: E402


def config1():
    P, Z, M, ptr = molecules_batch(seed=0)
    bi = oracle.batch_idx_from_ptr(ptr)
    B = len(ptr) - 1
    nm, nn, _ = oracle.nl_cell(P, None, None, ptr, 5.0, 32)
    cells = np.eye(3, dtype=np.float32)[None].repeat(B, 0)
    lj = oracle.lj_matrix(P, cells, nm, None, nn, bi, len(P), 0.01, 2.5, 5.0)
    Pf, Vf, Ff, Ef = nve(P, np.zeros_like(P), M, None, None, ptr, 5.0, 0.01, 2.5, 0.5, 100, K=32)
    np.savez_compressed(HERE / "config1_molecules.npz", positions=P, atomic_numbers=Z, masses=M, batch_ptr=ptr,
                        neighbor_matrix=nm, num_neighbors=nn, atomic_energies=lj["atomic_energies"],
                        forces=lj["forces"], energy=lj["energy"], final_positions=Pf, final_velocities=Vf,
                        final_forces=Ff, final_energy=Ef)


def triclinic():
    P, C, pb, ptr = periodic_batch(seed=53, n_systems=4, n_lo=20, n_hi=60, density=0.05, triclinic=True, spread=2.0)
    bi = oracle.batch_idx_from_ptr(ptr)
    K = 96
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, 6.0, K)
    assert nn.max() < K
    lj = oracle.lj_matrix(P, C, nm, sh, nn, bi, len(P), 0.01, 3.0, 6.0, virial=True)
    M = np.full(len(P), 39.95, dtype=np.float32)
    Pf, Vf, Ff, Ef, st, _ = fire(P, np.zeros_like(P), M, C, pb, ptr, 6.0, 0.01, 3.0, 0.1, 20, K=K)
    np.savez_compressed(HERE / "periodic_triclinic.npz", positions=P, cell=C, pbc=pb, batch_ptr=ptr, masses=M,
                        neighbor_matrix=nm, num_neighbors=nn, neighbor_matrix_shifts=sh,
                        atomic_energies=lj["atomic_energies"], forces=lj["forces"], energy=lj["energy"],
                        virials=lj["virials"], fire_positions=Pf, fire_velocities=Vf, fire_forces=Ff,
                        fire_energy=Ef, fire_dt=st["dt"], fire_alpha=st["alpha"],
                        fire_n_steps_positive=st["n_steps_positive"])


if __name__ == "__main__":
    config1()
    triclinic()
    for f in sorted(HERE.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")
