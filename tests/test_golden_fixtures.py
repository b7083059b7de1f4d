"""The committed fixtures of tests/golden (written by tests/golden/make_fixtures.py from the CPU
oracle): on the CPU the oracle must still reproduce them bit for bit; on the GPU the library is
checked against them without the oracle in the loop."""

from pathlib import Path

import numpy as np
import pytest
import torch

GOLDEN = Path(__file__).resolve().parent / "golden"
RTOL, ATOL = 1e-5, 1e-6


def load(name):
    with np.load(GOLDEN / name, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def canonical_rows(nm, nn, sh=None):
    """Sorted (i, j, sx, sy, sz) rows of the first nn[i] entries of every row."""
    K = nm.shape[1]
    ii, kk = np.nonzero(np.arange(K)[None, :] < np.minimum(nn, K)[:, None])
    s = sh[ii, kk] if sh is not None else np.zeros((len(ii), 3), np.int32)
    rows = np.concatenate([ii[:, None], nm[ii, kk][:, None], s], axis=1).astype(np.int64)
    return rows[np.lexsort(rows.T[::-1])]


def close(got, ref, what):
    got, ref = np.asarray(got, np.float64).reshape(ref.shape), np.asarray(ref, np.float64)
    err, tol = np.abs(got - ref), ATOL + RTOL * np.abs(ref)
    assert (err <= tol).all(), (what, float(err.max()))


def test_oracle_still_reproduces_the_fixtures():
    import oracle
    from _reference_loop import fire, nve

    g = load("config1_molecules.npz")
    P, M, ptr = g["positions"], g["masses"], g["batch_ptr"]
    bi = oracle.batch_idx_from_ptr(ptr)
    nm, nn, _ = oracle.nl_cell(P, None, None, ptr, 5.0, 32)
    assert np.array_equal(canonical_rows(nm, nn), canonical_rows(g["neighbor_matrix"], g["num_neighbors"]))
    cells = np.eye(3, dtype=np.float32)[None].repeat(len(ptr) - 1, 0)
    lj = oracle.lj_matrix(P, cells, nm, None, nn, bi, len(P), 0.01, 2.5, 5.0)
    assert np.array_equal(lj["forces"], g["forces"]) and np.array_equal(lj["energy"], g["energy"])
    Pf, Vf, Ff, Ef = nve(P, np.zeros_like(P), M, None, None, ptr, 5.0, 0.01, 2.5, 0.5, 100, K=32)
    assert np.array_equal(Pf, g["final_positions"]) and np.array_equal(Vf, g["final_velocities"])

    t = load("periodic_triclinic.npz")
    P, C, pb, ptr = t["positions"], t["cell"], t["pbc"], t["batch_ptr"]
    bi = oracle.batch_idx_from_ptr(ptr)
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, 6.0, 96)
    assert np.array_equal(canonical_rows(nm, nn, sh),
                          canonical_rows(t["neighbor_matrix"], t["num_neighbors"], t["neighbor_matrix_shifts"]))
    lj = oracle.lj_matrix(P, C, nm, sh, nn, bi, len(P), 0.01, 3.0, 6.0, virial=True)
    assert np.array_equal(lj["forces"], t["forces"]) and np.array_equal(lj["virials"], t["virials"])
    Pf, Vf, Ff, Ef, st, _ = fire(P, np.zeros_like(P), t["masses"], C, pb, ptr, 6.0, 0.01, 3.0, 0.1, 20, K=96)
    assert np.array_equal(Pf, t["fire_positions"]) and np.array_equal(st["dt"], t["fire_dt"])
    assert np.array_equal(st["n_steps_positive"], t["fire_n_steps_positive"])


def _batch(P, Z, M, ptr, C=None, pb=None):
    from nvalchemi_amd.data import AtomicData, Batch

    data = []
    for s in range(len(ptr) - 1):
        a0, a1 = int(ptr[s]), int(ptr[s + 1])
        kw = dict(atomic_masses=torch.from_numpy(M[a0:a1]), forces=torch.zeros(a1 - a0, 3), energy=torch.zeros(1, 1),
                  velocities=torch.zeros(a1 - a0, 3))
        if C is not None:
            kw["cell"], kw["pbc"] = torch.from_numpy(C[s]), torch.from_numpy(pb[s])
        data.append(AtomicData(torch.from_numpy(P[a0:a1]), torch.from_numpy(Z[a0:a1]), **kw))
    return Batch.from_data_list(data, device="cuda:0")


@pytest.mark.gpu
def test_gpu_config1_against_the_fixture():
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper
    from nvalchemi_amd.neighbors import compute_neighbors

    g = load("config1_molecules.npz")
    batch = _batch(g["positions"], g["atomic_numbers"], g["masses"], g["batch_ptr"])
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=2.5, cutoff=5.0)
    compute_neighbors(batch, config=model.model_config.neighbor_config)
    nm, nn = batch.neighbor_matrix.cpu().numpy(), batch.num_neighbors.cpu().numpy()
    assert np.array_equal(canonical_rows(nm, nn), canonical_rows(g["neighbor_matrix"], g["num_neighbors"]))
    out = model(batch)
    close(out["forces"].cpu().numpy(), g["forces"], "forces")
    close(out["energy"].cpu().numpy(), g["energy"], "energy")
    dyn = NVE(model, dt=0.5, hooks=model.make_neighbor_hooks())
    for _ in range(100):
        dyn.step(batch)
    close(batch.positions.cpu().numpy(), g["final_positions"], "positions after 100 steps")
    close(batch.velocities.cpu().numpy(), g["final_velocities"], "velocities after 100 steps")
    close(batch.forces.cpu().numpy(), g["final_forces"], "forces after 100 steps")
    close(batch.energy.cpu().numpy(), g["final_energy"], "energy after 100 steps")


@pytest.mark.gpu
def test_gpu_triclinic_against_the_fixture():
    from nvalchemi_amd import _lib
    from nvalchemi_amd.dynamics import FIRE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    t = load("periodic_triclinic.npz")
    P, C, pb, ptr = t["positions"], t["cell"], t["pbc"], t["batch_ptr"]
    N, B, K = len(P), len(C), t["neighbor_matrix"].shape[1]
    dev = "cuda:0"
    bi = torch.repeat_interleave(torch.arange(B, dtype=torch.int32), torch.from_numpy(np.diff(ptr)).long()).to(dev)
    nm = torch.full((N, K), N, dtype=torch.int32, device=dev)
    nn = torch.zeros(N, dtype=torch.int32, device=dev)
    sh = torch.zeros((N, K, 3), dtype=torch.int32, device=dev)
    tP, tC = torch.from_numpy(P).to(dev), torch.from_numpy(C).to(dev)
    _lib.nl_build(tP, tC, torch.from_numpy(pb).to(dev), torch.from_numpy(ptr).to(dev), bi, None, 6.0, K, False, 0,
                  nm, nn, sh)
    assert np.array_equal(canonical_rows(nm.cpu().numpy(), nn.cpu().numpy(), sh.cpu().numpy()),
                          canonical_rows(t["neighbor_matrix"], t["num_neighbors"], t["neighbor_matrix_shifts"]))
    e, f = torch.empty(N, device=dev), torch.empty((N, 3), device=dev)
    w, es = torch.empty((B, 9), device=dev), torch.empty(B, device=dev)
    # the fixture's own rows (another order than the GPU build's): results must not depend on it
    _lib.lj_energy_forces(tP, tC, torch.from_numpy(t["neighbor_matrix"]).to(dev),
                          torch.from_numpy(t["neighbor_matrix_shifts"]).to(dev),
                          torch.from_numpy(t["num_neighbors"]).to(dev), bi, N, 0.01, 3.0, 6.0, 0.0, False, e, f, w, es)
    close(f.cpu().numpy(), t["forces"], "forces")
    close(e.cpu().numpy(), t["atomic_energies"], "atomic energies")
    close(es.cpu().numpy(), t["energy"], "energy")
    wr = t["virials"].astype(np.float64)
    assert np.abs(w.cpu().numpy() - wr).max() <= ATOL + RTOL * np.abs(wr).max()
    batch = _batch(P, np.full(N, 18, np.int64), t["masses"], ptr, C, pb)
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=3.0, cutoff=6.0)
    dyn = FIRE(model, dt=0.1, hooks=model.make_neighbor_hooks(max_neighbors=K))
    for _ in range(20):
        dyn.step(batch)
    close(batch.positions.cpu().numpy(), t["fire_positions"], "positions after 20 FIRE steps")
    close(batch.forces.cpu().numpy(), t["fire_forces"], "forces after 20 FIRE steps")
    assert np.array_equal(dyn._state.n_steps_positive.cpu().numpy().ravel(), t["fire_n_steps_positive"])
    close(dyn._state.dt.cpu().numpy().ravel(), t["fire_dt"], "FIRE dt")
