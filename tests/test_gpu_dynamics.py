"""GPU end-to-end parity: the package's Batch / hooks / model / dynamics stack against step
loops driven by the CPU oracle on the same seeded inputs.

Tolerance: 1e-5 relative / 1e-6 absolute on positions, velocities, forces and energies over
the whole trajectory (the figure the task states for this path); neighbor data bit-exact as
canonical (i, j, shift) sets.
"""

import numpy as np
import pytest
import torch

import oracle
from _reference_loop import fire as ref_fire
from _reference_loop import nve as ref_nve
from _systems import fcc_boxes, molecules_batch, periodic_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-5, 1e-6


def make_batch(P, Z, M, C, pb, ptr, V=None):
    from nvalchemi_amd.data import AtomicData, Batch

    data = []
    for s in range(len(ptr) - 1):
        a0, a1 = int(ptr[s]), int(ptr[s + 1])
        kw = dict(atomic_masses=torch.from_numpy(M[a0:a1]), forces=torch.zeros(a1 - a0, 3),
                  energy=torch.zeros(1, 1))
        if V is not None:
            kw["velocities"] = torch.from_numpy(V[a0:a1])
        if C is not None:
            kw["cell"] = torch.from_numpy(C[s])
            kw["pbc"] = torch.from_numpy(pb[s])
        data.append(AtomicData(torch.from_numpy(P[a0:a1]), torch.from_numpy(Z[a0:a1]), **kw))
    return Batch.from_data_list(data, device=DEV)


def close(got, ref, what):
    got = got.detach().cpu().numpy().astype(np.float64).reshape(ref.shape)
    ref = ref.astype(np.float64)
    err = np.abs(got - ref)
    tol = ATOL + RTOL * np.abs(ref)
    assert (err <= tol).all(), (what, float(err.max()), float((err / tol).max()))


def test_config1_molecules_100_step_nve_trajectory():
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, Z, M, ptr = molecules_batch(seed=0)
    V = np.zeros_like(P)
    batch = make_batch(P, Z, M, None, None, ptr)
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=2.5, cutoff=5.0)
    dyn = NVE(model, dt=0.5, hooks=model.make_neighbor_hooks())
    checks = []

    def record(step, p, v, f, e):
        if step in (0, 1, 9, 49, 99):
            checks.append((step, p.copy(), v.copy(), f.copy(), e.copy()))

    ref_nve(P, V, M, None, None, ptr, 5.0, 0.01, 2.5, 0.5, 100, K=32, record=record)
    it = iter(checks)
    nxt = next(it)
    for step in range(100):
        dyn.step(batch)
        if nxt is not None and step == nxt[0]:
            close(batch.positions, nxt[1], f"positions@{step}")
            close(batch.velocities, nxt[2], f"velocities@{step}")
            close(batch.forces, nxt[3], f"forces@{step}")
            close(batch.energy, nxt[4], f"energy@{step}")
            nxt = next(it, None)
    assert dyn.step_count == 100 and nxt is None


def test_fcc_boxes_nve_trajectory_and_energy_conservation():
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=3, reps=3, a=3.6)
    N = len(P)
    rng = np.random.default_rng(1)
    M = np.full(N, 63.546, dtype=np.float32)
    V = rng.normal(0, 0.02, (N, 3)).astype(np.float32)
    Z = np.full(N, 29, dtype=np.int64)
    sig = (3.6 / np.sqrt(2)) / 2 ** (1 / 6)
    rc = 5.0  # below half the 10.8 A box
    batch = make_batch(P, Z, M, C, pb, ptr, V)
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=float(sig), cutoff=rc)
    dyn = NVE(model, dt=1.0, hooks=model.make_neighbor_hooks())
    dyn.run(batch, n_steps=100)
    rP, rV, rF, rE = ref_nve(P, V, M, C, pb, ptr, rc, 0.01, float(sig), 1.0, 100, K=96)
    close(batch.positions, rP, "positions")
    close(batch.velocities, rV, "velocities")
    close(batch.forces, rF, "forces")
    close(batch.energy, rE, "energy")
    # neighbor data on the batch is the oracle's, as a set (for the device's own final positions)
    ref = oracle.nl_brute(batch.positions.cpu().numpy(), C, pb, ptr, rc)
    got = oracle.matrix_to_edges(batch.neighbor_matrix.cpu().numpy(), batch.num_neighbors.cpu().numpy(),
                                 batch.neighbor_matrix_shifts.cpu().numpy())
    assert np.array_equal(got, ref)


def test_fire_relaxation_matches_oracle_and_reaches_the_minimum():
    from nvalchemi_amd.dynamics import FIRE, ConvergenceHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=3, n_boxes=2, reps=3, a=1.5496, jitter=0.03)  # nn distance ~ 1.096 sigma
    N = len(P)
    M = np.ones(N, dtype=np.float32)
    Z = np.full(N, 18, dtype=np.int64)
    batch = make_batch(P, Z, M, C, pb, ptr)
    model = LennardJonesModelWrapper(epsilon=1.0, sigma=1.0, cutoff=2.2)
    dyn = FIRE(model, dt=0.005, hooks=model.make_neighbor_hooks(),
               convergence_hook=ConvergenceHook.from_fmax(1e-3))
    n = 60
    for _ in range(n):
        dyn.step(batch)
    rP, rV, rF, rE, st, _ = ref_fire(P, np.zeros_like(P), M, C, pb, ptr, 2.2, 1.0, 1.0, 0.005, n, K=96)
    close(batch.positions, rP, "positions")
    close(batch.forces, rF, "forces")
    close(batch.energy, rE, "energy")
    assert np.array_equal(dyn._state.n_steps_positive.cpu().numpy(), st["n_steps_positive"])
    assert np.allclose(dyn._state.dt.cpu().numpy(), st["dt"], rtol=1e-6)
    # and it goes downhill
    e0 = ref_fire(P, np.zeros_like(P), M, C, pb, ptr, 2.2, 1.0, 1.0, 0.005, 1, K=96)[3]
    assert np.all(batch.energy.cpu().numpy().ravel() < e0)


def test_status_mask_freezes_converged_systems_like_the_oracle_loop():
    from nvalchemi_amd.dynamics import FIRE, ConvergenceHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    from _systems import ptr_from_counts

    parts = [fcc_boxes(seed=100 + s, n_boxes=1, reps=reps, a=1.5496, jitter=jit)
             for s, (reps, jit) in enumerate([(2, 0.005), (3, 0.05), (2, 0.02), (3, 0.01), (2, 0.08), (2, 0.002)])]
    P = np.concatenate([p[0] for p in parts])
    C = np.concatenate([p[1] for p in parts])
    pb = np.concatenate([p[2] for p in parts])
    ptr = ptr_from_counts([len(p[0]) for p in parts])
    N = len(P)
    M = np.ones(N, dtype=np.float32)
    Z = np.full(N, 18, dtype=np.int64)
    batch = make_batch(P, Z, M, C, pb, ptr)
    batch.status = torch.zeros(len(ptr) - 1, 1, dtype=torch.long, device=DEV)
    model = LennardJonesModelWrapper(epsilon=1.0, sigma=1.0, cutoff=2.2)
    tol = 1.0
    hook = ConvergenceHook.from_fmax(tol, source_status=0, target_status=1)
    dyn = FIRE(model, dt=0.005, hooks=model.make_neighbor_hooks() + [hook])
    n = 40
    for _ in range(n):
        dyn.step(batch)
    rP, rV, rF, rE, st, status = ref_fire(P, np.zeros_like(P), M, C, pb, ptr, 2.2, 1.0, 1.0, 0.005, n, K=96,
                                          fmax_tol=tol)
    assert np.array_equal(batch.status.cpu().numpy().ravel(), status)
    assert 0 < status.sum() < len(status), "the case must exercise both frozen and active systems"
    close(batch.positions, rP, "positions")
    close(batch.velocities, rV, "velocities")


def test_compute_neighbors_matrix_and_coo_and_hook_k_policy():
    from nvalchemi_amd.hooks import HookContext, NeighborListHook
    from nvalchemi_amd.models import NeighborConfig, NeighborListFormat
    from nvalchemi_amd.neighbors import compute_neighbors

    P, C, pb, ptr = periodic_batch(23, 4, 50, 200, 0.6)
    N = len(P)
    Z = np.ones(N, dtype=np.int64)
    M = np.ones(N, dtype=np.float32)
    ref = oracle.nl_brute(P, C, pb, ptr, 2.5)
    counts = np.bincount(ref[:, 0], minlength=N)

    batch = make_batch(P, Z, M, C, pb, ptr)
    compute_neighbors(batch, cutoff=2.5)  # estimate K=32 overflows at this density: the retry loop runs
    assert batch._neighbor_list_cutoff == 2.5
    K = batch.neighbor_matrix.shape[1]
    assert K > counts.max()
    got = oracle.matrix_to_edges(batch.neighbor_matrix.cpu().numpy(), batch.num_neighbors.cpu().numpy(),
                                 batch.neighbor_matrix_shifts.cpu().numpy())
    assert np.array_equal(got, ref)

    batch2 = make_batch(P, Z, M, C, pb, ptr)
    compute_neighbors(batch2, config=NeighborConfig(cutoff=2.5, format=NeighborListFormat.COO))
    nl = batch2.neighbor_list.cpu().numpy()
    sh = batch2.neighbor_list_shifts.cpu().numpy()
    assert nl.shape == (len(ref), 2) and sh.shape == (len(ref), 3) and batch2.neighbor_list.dtype == torch.int32
    assert np.array_equal(oracle.canonical_edges(np.concatenate([nl, sh], 1)), ref)
    assert np.all(np.diff(nl[:, 0]) >= 0), "row-major: sources ascending"
    assert np.array_equal(batch2.edge_ptr.cpu().numpy(), np.concatenate([[0], np.cumsum(counts)]))
    bi = oracle.batch_idx_from_ptr(ptr)
    assert np.array_equal(batch2.num_edges_per_graph.cpu().numpy(), np.bincount(bi[ref[:, 0]], minlength=4))
    with pytest.raises(ValueError):
        compute_neighbors(batch2)

    # hook: grows from the estimate, leaves a spare slot, results identical; second call reuses buffers
    hook = NeighborListHook(NeighborConfig(cutoff=2.5, format=NeighborListFormat.MATRIX))
    batch3 = make_batch(P, Z, M, C, pb, ptr)
    hook(HookContext(batch=batch3), None)
    assert hook._max_neighbors % 16 == 0 and hook._max_neighbors > counts.max()
    buf = hook._neighbor_matrix
    hook(HookContext(batch=batch3), None)
    assert hook._neighbor_matrix is buf and batch3.neighbor_matrix is buf
    got = oracle.matrix_to_edges(buf.cpu().numpy(), hook._num_neighbors.cpu().numpy(),
                                 hook._neighbor_matrix_shifts.cpu().numpy())
    assert np.array_equal(got, ref)
    # over-estimate is trimmed to ceil16(2*actual), never below the override
    hook2 = NeighborListHook(NeighborConfig(cutoff=2.5, format=NeighborListFormat.MATRIX), max_neighbors=512)
    hook2(HookContext(batch=batch3), None)
    assert hook2._max_neighbors == 512
    hook3 = NeighborListHook(NeighborConfig(cutoff=1.2, format=NeighborListFormat.MATRIX))
    hook3._max_neighbors_override = None
    b4 = make_batch(P, Z, M, C, pb, ptr)
    hook3(HookContext(batch=b4), None)
    actual = int(b4.num_neighbors.max())
    assert hook3._max_neighbors in (16, ((2 * actual + 15) // 16) * 16)


def test_non_periodic_batch_has_no_shift_key_and_lj_stress():
    from nvalchemi_amd.models import LennardJonesModelWrapper
    from nvalchemi_amd.neighbors import compute_neighbors

    P, Z, M, ptr = molecules_batch(seed=2)
    batch = make_batch(P, Z, M, None, None, ptr)
    compute_neighbors(batch, cutoff=5.0)
    assert getattr(batch, "neighbor_matrix_shifts", None) is None
    assert batch.neighbor_matrix.shape[1] == 32  # ceil16(max atoms per system)
    model = LennardJonesModelWrapper(0.01, 2.5, 5.0)
    out = model(batch)
    assert list(out.keys()) == ["energy", "forces"] and out["energy"].shape == (len(ptr) - 1, 1)

    Pp, C, pb, ptrp = fcc_boxes(seed=1, n_boxes=2, reps=3, a=0.95 * np.sqrt(2.0), jitter=0.02)
    b = make_batch(Pp, np.ones(len(Pp), dtype=np.int64), np.ones(len(Pp), dtype=np.float32), C, pb, ptrp)
    m2 = LennardJonesModelWrapper(1.0, 1.0, 1.3)
    m2.model_config.active_outputs = {"energy", "forces", "stress"}
    compute_neighbors(b, config=m2.model_config.neighbor_config)
    out = m2(b)
    bi = oracle.batch_idx_from_ptr(ptrp)
    ref = oracle.lj_matrix(Pp, C, b.neighbor_matrix.cpu().numpy(), b.neighbor_matrix_shifts.cpu().numpy(),
                           b.num_neighbors.cpu().numpy(), bi, len(Pp), 1.0, 1.0, 1.3, virial=True)
    vol = np.abs(np.linalg.det(C.astype(np.float64)))[:, None, None]
    exp = -ref["virials"].reshape(-1, 3, 3) / vol
    got = out["stress"].cpu().numpy()
    assert np.allclose(got, exp, rtol=1e-5, atol=1e-5 * np.abs(exp).max())
    assert np.all(np.diagonal(got, axis1=1, axis2=2) < 0)  # compressed: negative (tensile-positive convention)
    with pytest.raises(KeyError):  # a bare AtomicData carries no neighbor keys
        m2(b.get_data(0))


def test_one_md_step_replays_from_a_captured_graph():
    """Every entry point only enqueues kernels on the given stream (no allocation, no synchronisation,
    no memset nodes), so a whole step -- position update, neighbor build, pair kernel, velocity
    finalize -- can be captured once and replayed.  Replays are interleaved with eager work and
    synchronisations and checked against an eager run of the same steps."""
    from nvalchemi_amd import _lib

    P, C, pb, ptr = fcc_boxes(seed=3, n_boxes=6, reps=3, a=3.6)
    N, B, K, rc = len(P), len(ptr) - 1, 64, 4.5
    rng = np.random.default_rng(5)
    sig = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))

    def fresh():
        d = dict(pos=torch.from_numpy(P).to(DEV), vel=torch.from_numpy(rng.normal(0, 0.02, (N, 3)).astype(np.float32)).to(DEV),
                 frc=torch.zeros(N, 3, device=DEV), mass=torch.full((N,), 63.546, device=DEV),
                 dt=torch.full((B,), 0.1, device=DEV), cell=torch.from_numpy(C).to(DEV),
                 pbc=torch.from_numpy(pb).to(DEV), ptr=torch.from_numpy(ptr).to(DEV),
                 bidx=torch.from_numpy(oracle.batch_idx_from_ptr(ptr)).to(DEV),
                 nm=torch.full((N, K), N, dtype=torch.int32, device=DEV), nn=torch.zeros(N, dtype=torch.int32, device=DEV),
                 sh=torch.zeros(N, K, 3, dtype=torch.int32, device=DEV), e=torch.empty(N, device=DEV),
                 es=torch.empty(B, device=DEV))
        return d

    def step(d):
        _lib.vv_position_update(d["pos"], d["vel"], d["frc"], d["mass"], d["dt"], d["bidx"])
        _lib.nl_build(d["pos"], d["cell"], d["pbc"], d["ptr"], d["bidx"], None, rc, K, False, 0, d["nm"], d["nn"], d["sh"])
        _lib.lj_energy_forces(d["pos"], d["cell"], d["nm"], d["sh"], d["nn"], d["bidx"], N, 0.01, sig, rc, 0.0, False,
                              d["e"], d["frc"], None, d["es"])
        _lib.vv_velocity_finalize(d["vel"], d["frc"], d["mass"], d["dt"], d["bidx"])

    rng = np.random.default_rng(5)
    eager = fresh()
    rng = np.random.default_rng(5)
    graphed = fresh()
    step(eager)      # the first call sizes the workspaces (allocation happens outside the capture)
    step(graphed)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            step(graphed)
    torch.cuda.current_stream().wait_stream(side)
    # (the capture itself ran nothing: both copies have taken one step so far)
    for _ in range(5):
        g.replay()
        step(eager)
        scratch = torch.randn(1000, device=DEV).sum()  # unrelated eager work between replays
        torch.cuda.synchronize()
        for key in ("pos", "vel", "frc", "es"):
            assert torch.equal(graphed[key], eager[key]), key
        assert torch.equal(graphed["nn"], eager["nn"])
    assert float(scratch) == float(scratch)


def test_run_replays_captured_steps_bit_equal_to_eager_steps():
    """``run`` takes the steady-state steps of a plain NVE (no convergence criterion, hooks that are kernels
    only) by replaying one captured step.  100 steps that way, in two calls with unrelated eager work and
    synchronisations in between, against 100 eager steps of a second copy: positions, velocities and forces
    equal to the bit (per-system energies are float64 atomics summed in an order that varies from run to run:
    compared at the usual bar)."""
    from nvalchemi_amd.dynamics import NVE, DynamicsStage
    from nvalchemi_amd.hooks import WrapPeriodicHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=4, reps=3, a=3.6)
    N = len(P)
    rng = np.random.default_rng(1)
    M = np.full(N, 63.546, dtype=np.float32)
    V = rng.normal(0, 0.02, (N, 3)).astype(np.float32)
    Z = np.full(N, 29, dtype=np.int64)
    sig = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))

    def make(replay, skin):
        batch = make_batch(P, Z, M, C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=sig, cutoff=5.0)
        model.model_config.neighbor_config.skin = skin
        dyn = NVE(model, dt=1.0, hooks=model.make_neighbor_hooks() + [WrapPeriodicHook(stage=DynamicsStage.AFTER_POST_UPDATE)])
        dyn.graph_replay = replay
        return batch, dyn

    for skin in (0.0, 0.4):
        eager_batch, eager = make(False, skin)
        graph_batch, graphed = make(True, skin)
        eager.run(eager_batch, n_steps=100)
        graphed.run(graph_batch, n_steps=40)
        assert graphed._graph_state is not None and graphed._graph_state["graph"] is not None  # it was captured
        assert not graphed._graph_state["failed"]
        scratch = torch.randn(4096, device=DEV).square().sum()  # unrelated eager work between the two runs
        torch.cuda.synchronize()
        graphed.run(graph_batch, n_steps=60)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(scratch))
        assert eager.step_count == graphed.step_count == 100
        assert getattr(eager, "_graph_state", None) is None
        for name in ("positions", "velocities", "forces"):
            assert torch.equal(getattr(graph_batch, name), getattr(eager_batch, name)), (skin, name)
        close(graph_batch.energy, eager_batch.energy.cpu().numpy(), "energy")
        assert torch.equal(graph_batch.num_neighbors, eager_batch.num_neighbors)


def test_replayed_steps_of_a_large_system_and_of_fire_equal_eager_ones():
    """The same for the paths that keep state on the device from call to call: one system of more than 4096 atoms
    (the build leaves tile records for the pair kernel and skips zero shifts over zeros; its unit counter lives in
    two header slots taken in turn) under NVE, and FIRE (its sums live in two slots taken in turn) on small boxes."""
    from nvalchemi_amd.dynamics import FIRE, NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    def run_both(make, n_steps):
        out = []
        for replay in (False, True):
            batch, dyn = make()
            dyn.graph_replay = replay
            dyn.run(batch, n_steps=n_steps)
            torch.cuda.synchronize()
            assert (getattr(dyn, "_graph_state", None) is not None) == replay
            if replay:
                assert dyn._graph_state["graph"] is not None and not dyn._graph_state["failed"]
            out.append(batch)
        for name in ("positions", "velocities", "forces"):
            assert torch.equal(getattr(out[0], name), getattr(out[1], name)), name
        return out[1]

    # one box of 6000 atoms on a jittered lattice (so that no two atoms start close)
    n_side = 19
    L = n_side * 3.4
    g = np.random.default_rng(7)
    grid = np.stack(np.meshgrid(*[np.arange(n_side)] * 3, indexing="ij"), -1).reshape(-1, 3)[:6000]
    P = ((grid + 0.5) * 3.4 + g.normal(0, 0.15, (6000, 3))).astype(np.float32)
    C = (np.eye(3) * L).astype(np.float32)[None]
    pb = np.ones((1, 3), dtype=bool)
    ptr = np.array([0, 6000], dtype=np.int32)
    V = g.normal(0, 0.02, (6000, 3)).astype(np.float32)

    def big():
        batch = make_batch(P, np.full(6000, 18, dtype=np.int64), np.full(6000, 39.95, dtype=np.float32), C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.0, cutoff=7.0)
        return batch, NVE(model, dt=1.0, hooks=model.make_neighbor_hooks())

    batch = run_both(big, 30)
    assert getattr(batch, "_neighbor_pair_tiles", None) is not None  # (the tile path was the one taken)

    P2, C2, pb2, ptr2 = fcc_boxes(seed=4, n_boxes=3, reps=3, a=3.7, jitter=0.08)

    def relax():
        n = len(P2)
        batch = make_batch(P2, np.full(n, 29, dtype=np.int64), np.full(n, 63.546, dtype=np.float32), C2, pb2, ptr2,
                           np.zeros_like(P2))
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=float((3.6 / np.sqrt(2)) / 2 ** (1 / 6)), cutoff=5.0)
        return batch, FIRE(model, dt=0.5, hooks=model.make_neighbor_hooks())

    run_both(relax, 40)


def test_run_steps_eagerly_when_a_step_needs_the_host():
    """A convergence criterion ends a run from the host: such a dynamics is never captured."""
    from nvalchemi_amd.dynamics import FIRE, ConvergenceHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=2, n_boxes=2, reps=3, a=3.6)
    N = len(P)
    batch = make_batch(P, np.full(N, 29, dtype=np.int64), np.full(N, 63.546, dtype=np.float32), C, pb, ptr,
                       np.zeros_like(P))
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=float((3.6 / np.sqrt(2)) / 2 ** (1 / 6)), cutoff=5.0)
    dyn = FIRE(model, dt=0.5, hooks=model.make_neighbor_hooks(), convergence_hook=ConvergenceHook.from_fmax(1e-3))
    dyn.run(batch, n_steps=10)
    assert getattr(dyn, "_graph_state", None) is None


def test_hook_leaves_the_cell_order_for_large_systems_and_the_model_uses_it():
    from nvalchemi_amd.hooks import HookContext
    from nvalchemi_amd.models import LennardJonesModelWrapper

    rng = np.random.default_rng(3)
    n_big, n_small, rho = 6000, 300, 0.8
    P, C, ptr = [], [], [0]
    for n in (n_small, n_big):
        L = (n / rho) ** (1 / 3)
        P.append(rng.uniform(0, L, (n, 3)).astype(np.float32))
        C.append(np.eye(3, dtype=np.float32) * L)
        ptr.append(ptr[-1] + n)
    P, C, ptr = np.concatenate(P), np.stack(C), np.array(ptr, np.int32)
    N = len(P)
    pb = np.ones((2, 3), bool)
    batch = make_batch(P, np.full(N, 18, np.int64), np.ones(N, np.float32), C, pb, ptr)
    model = LennardJonesModelWrapper(epsilon=1.0, sigma=0.5, cutoff=2.5)
    hook = model.make_neighbor_hooks()[0]
    hook(HookContext(batch=batch), None)
    order = batch._neighbor_row_order
    assert order is not None and order.dtype == torch.int32 and order.shape == (N,)
    o = order.cpu().numpy()
    for s in range(2):  # a permutation of each system's own range
        assert np.array_equal(np.sort(o[ptr[s]:ptr[s + 1]]), np.arange(ptr[s], ptr[s + 1]))
    with_order = model(batch)
    object.__setattr__(batch, "_neighbor_row_order", None)
    without = model(batch)
    assert torch.equal(with_order["forces"], without["forces"])
    assert torch.allclose(with_order["energy"], without["energy"], rtol=1e-6, atol=0)
    # a batch of small systems gets no order
    small = make_batch(P[:n_small], np.full(n_small, 18, np.int64), np.ones(n_small, np.float32), C[:1], pb[:1],
                       np.array([0, n_small], np.int32))
    hook2 = model.make_neighbor_hooks()[0]
    hook2(HookContext(batch=small), None)
    assert getattr(small, "_neighbor_row_order", None) is None


def test_masked_update_moves_only_the_selected_systems():
    """``masked_update`` / ``_masked_pre_update`` / ``_masked_post_update``
    (nvalchemi/dynamics/base.py:2085-2212): selected systems advance exactly as in an unmasked
    update, the others keep positions and velocities -- through the kernels' own mask (NVE) and
    through the save-and-restore route of integrators that do not take one."""
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = periodic_batch(seed=77, n_systems=5, n_lo=40, n_hi=90, density=0.5)
    rng = np.random.default_rng(1)
    V = rng.normal(0, 0.3, P.shape).astype(np.float32)
    F = rng.normal(0, 1.0, P.shape).astype(np.float32)
    Z = np.full(len(P), 18, dtype=np.int64)
    M = np.full(len(P), 39.95, dtype=np.float32)
    mask = torch.tensor([True, False, True, True, False], device=DEV)
    node = mask[torch.repeat_interleave(torch.arange(5, device=DEV), torch.as_tensor(np.diff(ptr), device=DEV))]

    class PlainNVE(NVE):
        _honors_active_mask = False  # forces the save-and-restore route

    for cls in (NVE, PlainNVE):
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=3.0, cutoff=6.0)
        full, part, halves = (make_batch(P, Z, M, C, pb, ptr, V=V) for _ in range(3))
        for b in (full, part, halves):
            b.forces.copy_(torch.from_numpy(F))
        dyn = cls(model, dt=1.0)
        dyn.masked_update(full, torch.ones(5, dtype=torch.bool, device=DEV))
        dyn.masked_update(part, mask)
        dyn._masked_pre_update(halves, mask)
        dyn._masked_post_update(halves, mask)
        p0, v0 = torch.from_numpy(P).to(DEV), torch.from_numpy(V).to(DEV)
        for b in (part, halves):
            assert torch.equal(b.positions[node], full.positions[node]) and torch.equal(b.velocities[node], full.velocities[node])
            assert torch.equal(b.positions[~node], p0[~node]) and torch.equal(b.velocities[~node], v0[~node])
        assert not torch.equal(full.positions[~node], p0[~node])


def test_fused_stage_relax_then_md_equals_each_system_on_its_own():
    """``FIRE + NVE`` as one ``FusedStage`` (nvalchemi/dynamics/base.py:2504-3337): every system
    relaxes until its forces fall below the threshold, then runs its budget of MD steps, then
    rests.  Systems do not interact, so the fused batch must reproduce each system taken through
    the same two dynamics alone."""
    from nvalchemi_amd.dynamics import FIRE, NVE, ConvergenceHook, FusedStage
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=5, n_boxes=4, reps=3, a=5.4, jitter=0.0)
    rng = np.random.default_rng(3)
    for s, amp in enumerate((0.02, 0.10, 0.25, 0.05)):  # different distances from the minimum
        P[ptr[s]:ptr[s + 1]] += rng.normal(0, amp, (ptr[s + 1] - ptr[s], 3)).astype(np.float32)
    Z = np.full(len(P), 18, dtype=np.int64)
    M = np.full(len(P), 39.95, dtype=np.float32)
    tol, md_steps, cap = 0.02, 5, 400

    def dynamics():
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
        relax = FIRE(model, dt=1.0, convergence_hook=ConvergenceHook.from_fmax(tol))
        md = NVE(model, dt=2.0, n_steps=md_steps)
        return model, relax, md

    model, relax, md = dynamics()
    fused = relax + md
    assert isinstance(fused, FusedStage) and fused.exit_status == 2 and [c for c, _ in fused.sub_stages] == [0, 1]
    for h in model.make_neighbor_hooks():
        fused.register_hook(h)
    batch = make_batch(P, Z, M, C, pb, ptr, V=np.zeros_like(P))
    graduated_at = {}
    fused._ensure_bookkeeping_fields(batch)
    fused._call_hooks(fused._stage_type.BEFORE_COMPUTE, batch)
    fused.compute(batch)
    for step in range(cap):
        batch, done = fused.step(batch)
        if done is not None:
            for s in done.tolist():
                graduated_at[s] = step
        if FusedStage.all_complete(batch, fused.exit_status):
            break
    assert sorted(graduated_at) == [0, 1, 2, 3] and len(set(graduated_at.values())) > 1
    assert batch.status.view(-1).tolist() == [2, 2, 2, 2]

    for s in range(4):
        a0, a1 = int(ptr[s]), int(ptr[s + 1])
        one_ptr = np.array([0, a1 - a0], dtype=np.int32)
        model, relax, md = dynamics()
        b = make_batch(P[a0:a1], Z[a0:a1], M[a0:a1], C[s:s + 1], pb[s:s + 1], one_ptr, V=np.zeros((a1 - a0, 3), np.float32))
        hooks = model.make_neighbor_hooks()
        for h in hooks:
            relax.register_hook(h)
            md.register_hook(h)
        relax._call_hooks(relax._stage_type.BEFORE_COMPUTE, b)
        relax.compute(b)
        steps = 0
        while True:
            _, conv = relax.step(b)
            steps += 1
            if conv is not None:
                break
            assert steps < cap
        # the step budget of a sub-stage counts the step in which a system arrives
        # (nvalchemi/dynamics/base.py:3023-3028 reads the status after the migration)
        for _ in range(md_steps - 1):
            md.step(b)
        assert graduated_at[s] == steps + md_steps - 2, (s, graduated_at[s], steps)
        close(batch.positions[a0:a1], b.positions.cpu().numpy(), f"positions of system {s}")
        close(batch.velocities[a0:a1], b.velocities.cpu().numpy(), f"velocities of system {s}")

    # run(): the same through the loop of the class, and a finished batch stays put
    model, relax, md = dynamics()
    fused2 = FusedStage([(0, relax), (1, md)], hooks=model.make_neighbor_hooks())
    batch2 = fused2.run(make_batch(P, Z, M, C, pb, ptr, V=np.zeros_like(P)), n_steps=cap)
    assert torch.equal(batch2.positions, batch.positions) and torch.equal(batch2.velocities, batch.velocities)
    frozen = batch2.positions.clone()
    fused2.step(batch2)
    assert torch.equal(batch2.positions, frozen)
    with pytest.raises(ValueError):
        fused2.run(None)
    with pytest.raises(TypeError):
        fused2 + 3


class _ListSampler:
    """The sampler protocol ``refill_check`` needs, over a list of systems
    (nvalchemi/dynamics/sampler.py:261-516: initial batch, budgeted replacements, exhaustion)."""

    def __init__(self, systems, batch_size):
        self._systems = list(systems)
        self.max_batch_size = batch_size
        self.max_atoms = None
        self.max_edges = None
        self.handed_out = 0

    def _take(self, n):
        out = self._systems[:n]
        self._systems = self._systems[n:]
        self.handed_out += len(out)
        return out

    def build_initial_batch(self):
        from nvalchemi_amd.data import Batch

        return Batch.from_data_list(self._take(self.max_batch_size), device=DEV)

    def request_replacements_budget(self, atom_budget=None, edge_budget=None, max_count=None):
        return self._take(max_count if max_count is not None else 1)

    @property
    def exhausted(self):
        return not self._systems


def test_fused_stage_refills_finished_systems_from_a_sampler():
    """In-flight batching (nvalchemi/dynamics/base.py:1957-2083, 3162-3265): seven systems go
    through a batch of three slots; each is relaxed exactly as it would be alone, finished systems
    are replaced, integrator state and bookkeeping fields follow their systems."""
    from nvalchemi_amd.data import AtomicData
    from nvalchemi_amd.dynamics import FIRE, ConvergenceHook, FusedStage
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=9, n_boxes=7, reps=3, a=5.4, jitter=0.0)
    rng = np.random.default_rng(4)
    amps = (0.02, 0.2, 0.05, 0.12, 0.03, 0.3, 0.08)
    for s, amp in enumerate(amps):
        P[ptr[s]:ptr[s + 1]] += rng.normal(0, amp, (ptr[s + 1] - ptr[s], 3)).astype(np.float32)
    tol = 0.02

    def system(s):
        a0, a1 = int(ptr[s]), int(ptr[s + 1])
        n = a1 - a0
        return AtomicData(torch.from_numpy(P[a0:a1]), torch.full((n,), 18), atomic_masses=torch.full((n,), 39.95),
                          forces=torch.zeros(n, 3), energy=torch.zeros(1, 1), velocities=torch.zeros(n, 3),
                          cell=torch.from_numpy(C[s]), pbc=torch.from_numpy(pb[s]),
                          system_id=torch.full((1, 1), s, dtype=torch.long))

    def relaxer():
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
        return model, FIRE(model, dt=1.0, convergence_hook=ConvergenceHook.from_fmax(tol))

    # each system alone: the steps it needs and where it ends
    alone = {}
    for s in range(7):
        from nvalchemi_amd.data import Batch

        model, relax = relaxer()
        for h in model.make_neighbor_hooks():
            relax.register_hook(h)
        b = Batch.from_data_list([system(s)], device=DEV)
        if s < 3:
            # the first batch is evaluated before its first step; a newcomer is not: it takes its
            # first step with the zero forces it arrives with (FIRE shortens its time step there)
            relax._call_hooks(relax._stage_type.BEFORE_COMPUTE, b)
            relax.compute(b)
        steps = 0
        while True:
            _, conv = relax.step(b)
            steps += 1
            if conv is not None:
                break
            assert steps < 500
        alone[s] = (steps, b.positions.cpu().numpy())
    assert len({v[0] for v in alone.values()}) > 2

    model, relax = relaxer()
    sampler = _ListSampler([system(s) for s in range(7)], batch_size=3)
    finished = {}

    class Collect:
        frequency = 1
        stage = FusedStage._stage_type.AFTER_STEP

        def __call__(self, ctx, stage):
            b = ctx.batch
            done = torch.where(b.status.view(-1) >= 1)[0].tolist()
            for k in done:
                sid = int(b.system_id.view(-1)[k])
                if sid not in finished:
                    a0, a1 = int(b.batch_ptr[k]), int(b.batch_ptr[k + 1])
                    finished[sid] = b.positions[a0:a1].cpu().numpy()

    fused = FusedStage([(0, relax)], hooks=model.make_neighbor_hooks(), sampler=sampler, refill_frequency=1)
    fused.register_fused_hook(Collect())
    out = fused.run(None, n_steps=2000)
    assert out is None and fused.done and sampler.exhausted and sampler.handed_out == 7
    assert sorted(finished) == list(range(7))
    for s in range(7):
        ref = alone[s][1]
        err = np.abs(finished[s].astype(np.float64) - ref)
        assert (err <= ATOL + RTOL * np.abs(ref)).all(), (s, float(err.max()))


def test_nvt_langevin_thermalises_an_lj_crystal():
    """``NVTLangevin`` on 4 FCC argon boxes started at rest: the kinetic temperature settles at the
    target (equipartition over 2000 atoms, a few per cent), different seeds give different
    trajectories, the same seed the same one, and the run follows the oracle step loop."""
    from nvalchemi_amd.dynamics import NVTLangevin
    from nvalchemi_amd.dynamics.hooks import temperature_per_graph
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=2, n_boxes=4, reps=5, a=5.4, jitter=0.02)
    N = len(P)
    Z = np.full(N, 18, dtype=np.int64)
    M = np.full(N, 39.95, dtype=np.float32)
    T_target = 80.0

    def run(seed, steps):
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
        dyn = NVTLangevin(model, dt=4.0, temperature=T_target, friction=0.02, random_seed=seed,
                          hooks=model.make_neighbor_hooks())
        batch = make_batch(P, Z, M, C, pb, ptr, V=np.zeros_like(P))
        temps = []
        for k in range(steps):
            dyn.step(batch)
            if k >= steps // 2:
                temps.append(temperature_per_graph(batch.velocities, batch.atomic_masses, batch.batch_idx, 4,
                                                   batch.num_nodes_per_graph).mean().item())
        return batch, float(np.mean(temps))

    b1, t1 = run(7, 400)
    assert abs(t1 / T_target - 1) < 0.06, t1
    b2, _ = run(7, 400)
    assert torch.equal(b1.positions, b2.positions)
    b3, _ = run(8, 400)
    assert not torch.equal(b1.positions, b3.positions)

    # a short run against the oracle loop (pre: half step; neighbor list + LJ; post: half kick)
    from _reference_loop import FS_PER_INTERNAL_TIME, build_and_eval

    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
    dyn = NVTLangevin(model, dt=2.0, temperature=T_target, friction=0.05, random_seed=3, hooks=model.make_neighbor_hooks())
    batch = make_batch(P, Z, M, C, pb, ptr, V=np.zeros_like(P))
    p, v, f = P.copy(), np.zeros_like(P), np.zeros_like(P)
    bi = oracle.batch_idx_from_ptr(ptr)
    dt = np.full(4, np.float32(2.0 / FS_PER_INTERNAL_TIME), np.float32)
    kT = np.full(4, np.float32(T_target * 8.617333262e-5), np.float32)
    gamma = np.full(4, np.float32(0.05 * FS_PER_INTERNAL_TIME), np.float32)
    K = 96
    for step in range(10):
        dyn.step(batch)
        oracle.langevin_half_step(p, v, f, M, dt, kT, gamma, 3 + step, bi)
        out, K = build_and_eval(p, C, pb, ptr, bi, 8.0, 0.0104, 3.4, K)
        f = out["forces"]
        oracle.vv_post(v, f, M, dt, bi)
    close(batch.positions, p, "positions after 10 Langevin steps")
    close(batch.velocities, v, "velocities after 10 Langevin steps")


def test_nvt_nose_hoover_follows_the_oracle_loop_thermalises_and_conserves_its_energy():
    """``NVTNoseHoover`` on 4 FCC argon boxes: 20 steps against the oracle step loop (chain - kick -
    drift | neighbor list + LJ | kick - chain); over a longer run the extended energy
    KE + PE + sum Q u^2/2 + N_f kT eta_1 + kT sum_{k>1} eta_k stays put while the thermostat moves
    energy in and out, and the kinetic temperature settles at the target."""
    from _reference_loop import FS_PER_INTERNAL_TIME, build_and_eval
    from nvalchemi_amd.dynamics import NVTNoseHoover
    from nvalchemi_amd.dynamics.hooks import kinetic_energy_per_graph, temperature_per_graph
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=2, n_boxes=4, reps=4, a=5.4, jitter=0.02)
    N = len(P)
    Z = np.full(N, 18, dtype=np.int64)
    M = np.full(N, 39.95, dtype=np.float32)
    rng = np.random.default_rng(5)
    T_target = np.array([60.0, 80.0, 100.0, 120.0], np.float32)
    kB = 8.617333262e-5
    bi = oracle.batch_idx_from_ptr(ptr)
    V0 = (rng.normal(0, 1, (N, 3)) * np.sqrt(kB * 40.0 / M)[:, None]).astype(np.float32)  # 40 K everywhere
    chain = 3

    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
    dyn = NVTNoseHoover(model, dt=2.0, temperature=torch.from_numpy(T_target), thermostat_time=50.0,
                        chain_length=chain, yoshida_order=5, hooks=model.make_neighbor_hooks())
    batch = make_batch(P, Z, M, C, pb, ptr, V=V0)
    p, v, f = P.copy(), V0.copy(), np.zeros_like(P)
    dt = np.full(4, np.float32(2.0 / FS_PER_INTERNAL_TIME), np.float32)
    kT = (T_target * np.float32(kB)).astype(np.float32)
    tau = np.full(4, np.float32(50.0 / FS_PER_INTERNAL_TIME), np.float32)
    ndof = (3 * np.diff(ptr)).astype(np.float32)
    Q = oracle.nhc_masses(kT, tau, ndof, chain)
    eta, u = np.zeros((4, chain), np.float32), np.zeros((4, chain), np.float32)
    K = 96
    for step in range(20):
        dyn.step(batch)
        oracle.nhc_chain_update(v, M, eta, u, Q, kT, dt, ndof, bi, yoshida_order=5)
        oracle.vv_post(v, f, M, dt, bi)
        oracle.nhc_position_update(p, v, dt, bi)
        out, K = build_and_eval(p, C, pb, ptr, bi, 8.0, 0.0104, 3.4, K)
        f = out["forces"]
        oracle.vv_post(v, f, M, dt, bi)
        oracle.nhc_chain_update(v, M, eta, u, Q, kT, dt, ndof, bi, yoshida_order=5)
    close(batch.positions, p, "positions after 20 Nose-Hoover steps")
    close(batch.velocities, v, "velocities after 20 Nose-Hoover steps")
    close(dyn._state.nhc_eta, eta, "chain positions")
    close(dyn._state.nhc_eta_dot, u, "chain velocities")
    assert np.allclose(dyn._state.nhc_Q.cpu().numpy(), Q, rtol=1e-6)

    # ---- a longer run: the conserved quantity and the temperature
    def extended(b, d):
        ke = kinetic_energy_per_graph(b.velocities, b.atomic_masses, b.batch_idx, 4).double().cpu().numpy().reshape(4)
        pe = b.energy.double().cpu().numpy().reshape(4)
        s = d._state
        qu = 0.5 * (s.nhc_Q.double() * s.nhc_eta_dot.double() ** 2).sum(1).cpu().numpy()
        e = s.nhc_eta.double().cpu().numpy()
        return ke + pe + qu + ndof * kT.astype(np.float64) * e[:, 0] + kT.astype(np.float64) * e[:, 1:].sum(1), ke

    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
    dyn = NVTNoseHoover(model, dt=2.0, temperature=torch.from_numpy(T_target), thermostat_time=50.0,
                        hooks=model.make_neighbor_hooks())
    batch = make_batch(P, Z, M, C, pb, ptr, V=V0)
    dyn.step(batch)
    h0, ke0 = extended(batch, dyn)
    temps, drift = [], 0.0
    steps = 1500
    for k in range(steps):
        dyn.step(batch)
        if k % 50 == 49:
            h, _ = extended(batch, dyn)
            drift = max(drift, float(np.abs(h - h0).max()))
        if k >= steps // 2:
            temps.append(temperature_per_graph(batch.velocities, batch.atomic_masses, batch.batch_idx, 4,
                                               batch.num_nodes_per_graph).cpu().numpy().reshape(4))
    mean_t = np.mean(temps, axis=0)
    assert np.all(np.abs(mean_t / T_target - 1) < 0.08), mean_t
    # the heat taken up is of the order of N_f k (T_target - 20 K) / 2 ~ 1 eV per box; the sum moves by far less
    taken = np.abs(ndof * kT * dyn._state.nhc_eta[:, 0].double().cpu().numpy())
    assert taken.min() > 0.2 and drift < 0.01 * taken.min(), (drift, taken)


def test_fire2_relaxation_matches_oracle_and_reaches_the_minimum():
    """``FIRE2`` through the package API on jittered FCC argon boxes: the first 40 steps against the
    oracle loop (step on the old forces | neighbor list + LJ), then on to fmax < 1e-3 eV/A, at the
    energy of the perfect crystal."""
    from _reference_loop import build_and_eval
    from nvalchemi_amd.dynamics import FIRE2, ConvergenceHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=6, n_boxes=3, reps=3, a=5.26, jitter=0.08)
    N = len(P)
    Z = np.full(N, 18, dtype=np.int64)
    M = np.full(N, 39.95, dtype=np.float32)
    bi = oracle.batch_idx_from_ptr(ptr)
    params = dict(delaystep=5, tmax=3.0, tmin=0.05, maxstep=0.1)
    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
    dyn = FIRE2(model, dt=1.0, hooks=model.make_neighbor_hooks(), convergence_hook=ConvergenceHook.from_fmax(1e-3),
                **params)
    batch = make_batch(P, Z, M, C, pb, ptr, V=np.zeros_like(P))
    K = 96
    p, v = P.copy(), np.zeros_like(P)
    alpha, dt, cnt = np.full(3, 0.09, np.float32), np.full(3, 1.0, np.float32), np.zeros(3, np.int32)
    # the forces of the start: the package evaluates them in run(); here by hand on both sides
    out, K = build_and_eval(p, C, pb, ptr, bi, 8.0, 0.0104, 3.4, K)
    f = out["forces"]
    dyn._call_hooks(dyn._stage_type.BEFORE_COMPUTE, batch)
    dyn.compute(batch)
    for step in range(40):
        dyn.step(batch)
        oracle.fire2_step(p, v, f, bi, alpha, dt, cnt, **params)
        out, K = build_and_eval(p, C, pb, ptr, bi, 8.0, 0.0104, 3.4, K)
        f = out["forces"]
    close(batch.positions, p, "positions after 40 FIRE2 steps")
    close(batch.forces, f, "forces after 40 FIRE2 steps")
    assert np.array_equal(dyn._state.nsteps_inc.cpu().numpy(), cnt)
    assert np.allclose(dyn._state.dt.cpu().numpy(), dt, rtol=1e-6)
    e40 = batch.energy.cpu().numpy().reshape(3).copy()
    converged = None
    for step in range(600):
        _, converged = dyn.step(batch)
        if converged is not None and converged.numel() == 3:
            break
    assert converged is not None and converged.numel() == 3, step
    e = batch.energy.cpu().numpy().reshape(3)
    assert np.all(e <= e40 + 1e-6)
    # the perfect lattice is the minimum: every box ends at the same energy per atom
    per_atom = e / np.diff(ptr)
    assert np.ptp(per_atom) < 2e-6 * abs(per_atom.mean()) + 1e-7, per_atom
    fm = np.linalg.norm(batch.forces.cpu().numpy(), axis=1).max()
    assert fm < 1e-3


def test_integrator_state_follows_its_systems_through_a_refill():
    """Restating test/dynamics/test_state_management.py:633-849: after ``refill_check`` the per-system
    state has one row per system of the new batch -- the rows of the systems that stay, in order and
    unchanged, then fresh rows for the newcomers -- for a plain integrator and for every sub-stage of
    a fused stage; when nothing is left the state is dropped and the run is done."""
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.dynamics import FIRE, NVE, FusedStage
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=3, n_boxes=5, reps=2, a=5.4, jitter=0.1)

    def system(s):
        a0, a1 = int(ptr[s]), int(ptr[s + 1])
        n = a1 - a0
        return AtomicData(torch.from_numpy(P[a0:a1]), torch.full((n,), 18), atomic_masses=torch.full((n,), 39.95),
                          forces=torch.zeros(n, 3), energy=torch.zeros(1, 1), velocities=torch.zeros(n, 3),
                          cell=torch.from_numpy(C[s]), pbc=torch.from_numpy(pb[s]))

    def batch_of(ids):
        b = Batch.from_data_list([system(s) for s in ids], device=DEV)
        b["status"] = torch.zeros(len(ids), 1, dtype=torch.long, device=DEV)
        return b

    def fire_with(replacements):
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=5.0)
        sampler = _ListSampler(replacements, batch_size=3)
        return FIRE(model, dt=1.0, hooks=model.make_neighbor_hooks(), sampler=sampler)

    # no replacement: a row less, the others as they were
    dyn = fire_with([])
    batch = batch_of([0, 1, 2])
    for _ in range(6):
        dyn.step(batch)
    s = dyn._state
    assert s.num_graphs == 3 and int(s.n_steps_positive.max()) > 0
    before = {k: getattr(s, k)[1:].clone() for k in ("alpha", "dt", "n_steps_positive")}
    batch.status[0] = 1
    result = dyn.refill_check(batch, exit_status=1)
    assert result.num_graphs == 2 and dyn._state.num_graphs == 2 and dyn.done is False
    for k, v in before.items():
        assert torch.equal(getattr(dyn._state, k), v), k
    dyn.step(result)  # and the integrator goes on with it

    # one replacement: same size; the newcomer starts from the defaults
    dyn = fire_with([system(3)])
    batch = batch_of([0, 1])
    for _ in range(8):
        dyn.step(batch)
    kept_alpha = dyn._state.alpha[1].clone()
    batch.status[0] = 1
    result = dyn.refill_check(batch, exit_status=1)
    assert result.num_graphs == 2 and dyn._state.num_graphs == 2
    assert torch.equal(dyn._state.alpha[0], kept_alpha)
    assert int(dyn._state.n_steps_positive[-1]) == 0 and float(dyn._state.alpha[-1]) == pytest.approx(dyn.alpha_start)
    assert float(dyn._state.dt[-1]) == 1.0
    dyn.step(result)

    # everything leaves and nothing comes: no state, done
    dyn = fire_with([])
    batch = batch_of([0, 1])
    dyn.step(batch)
    batch.status[:] = 1
    assert dyn.refill_check(batch, exit_status=1) is None and not hasattr(dyn, "_state") and dyn.done is True

    # a fused stage keeps the state of each of its sub-stages in step
    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=5.0)
    relax, md = FIRE(model, dt=1.0), NVE(model, dt=1.0)
    fused = FusedStage([(0, relax), (1, md)], hooks=model.make_neighbor_hooks(),
                       sampler=_ListSampler([system(3), system(4)], batch_size=3), exit_status=2)
    batch = batch_of([0, 1, 2])
    batch.status[1] = 1  # (a sub-stage makes its state the first time a system carries its code)
    fused.step(batch)
    assert relax._state.num_graphs == 3 and md._state.num_graphs == 3
    batch.status[1] = 2
    result = fused.refill_check(batch, exit_status=2)
    assert result.num_graphs == 3 and relax._state.num_graphs == 3 and md._state.num_graphs == 3
    fused.step(result)
    result.status[:] = 2
    result = fused.refill_check(result, exit_status=2)
    assert result.num_graphs == 1 and relax._state.num_graphs == 1 and md._state.num_graphs == 1
    result.status[:] = 2
    assert fused.refill_check(result, exit_status=2) is None and fused.done
    assert not hasattr(relax, "_state") and not hasattr(md, "_state")


def test_steps_inside_the_stream_context_run_on_its_stream_and_give_the_same_trajectory():
    """``with dynamics:`` (nvalchemi/dynamics/base.py:686-742, 2790-2840): a stream of its own becomes
    current, the kernels of the steps inside go to it (the library launches on the current stream),
    sub-stages of a fused stage report the same stream, and the trajectory is the one of the default
    stream bit for bit."""
    from nvalchemi_amd.dynamics import NVE, FusedStage
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=8, n_boxes=3, reps=3, a=5.4, jitter=0.05)
    N = len(P)
    Z = np.full(N, 18, dtype=np.int64)
    M = np.full(N, 39.95, dtype=np.float32)

    def run(in_context):
        model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
        dyn = NVE(model, dt=2.0, hooks=model.make_neighbor_hooks())
        batch = make_batch(P, Z, M, C, pb, ptr, V=np.zeros_like(P))
        torch.cuda.synchronize()
        if in_context:
            default = torch.cuda.current_stream()
            with dyn as entered:
                assert entered is dyn and dyn.stream is not None
                assert torch.cuda.current_stream() == dyn.stream and dyn.stream != default
                for _ in range(10):
                    dyn.step(batch)
                dyn.stream.synchronize()
            assert dyn.stream is None and torch.cuda.current_stream() == default
        else:
            for _ in range(10):
                dyn.step(batch)
            torch.cuda.synchronize()
        return batch.positions.clone(), batch.velocities.clone()

    p0, v0 = run(False)
    p1, v1 = run(True)
    assert torch.equal(p0, p1) and torch.equal(v0, v1)
    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=8.0)
    a, b = NVE(model, dt=1.0), NVE(model, dt=1.0)
    fused = FusedStage([(0, a), (1, b)])
    with fused:
        assert fused.stream is not None and a.stream is fused.stream and b.stream is fused.stream
    assert fused.stream is None and a.stream is None and b.stream is None


def test_status_migration_in_one_launch_equals_the_torch_expression():
    """nvamd_status_migrate against ``status[(values <= thr) & (status == source)] = target`` written out in Torch
    (nvalchemi/dynamics/base.py:2459-2502), on values that include the threshold itself, -inf (a system without
    atoms), +inf and NaN; float32 and float64 values; and ConvergenceHook with one force criterion (the one launch)
    against the same hook with a second, always-true criterion (the general Torch path)."""
    from nvalchemi_amd import _lib
    from nvalchemi_amd.dynamics import ConvergenceHook
    from nvalchemi_amd.hooks._context import DynamicsContext

    g = torch.Generator().manual_seed(3)
    M = 1000
    for dtype in (torch.float32, torch.float64):
        values = torch.rand(M, generator=g, dtype=dtype) * 0.1
        values[:6] = torch.tensor([0.05, float("-inf"), float("inf"), float("nan"), 0.05000001, 0.04999999], dtype=dtype)
        status = torch.randint(0, 3, (M + 7,), generator=g, dtype=torch.int64)
        status[:6] = 1
        want = status.clone()
        thr = torch.tensor(0.05, dtype=dtype)
        pick = (values <= thr) & (want[:M] == 1)
        want[:M][pick] = 5
        got = status.to(DEV)
        _lib.status_migrate(values.to(DEV), 0.05, got, 1, 5)
        assert torch.equal(got.cpu(), want), dtype
        assert want[0] == 5 and want[1] == 5 and want[2] == 1 and want[3] == 1 and want[5] == 5
    with pytest.raises(ValueError):
        _lib.status_migrate(values.to(DEV), 0.05, status[:10].to(DEV), 1, 5)
    with pytest.raises(ValueError):
        _lib.status_migrate(values.to(DEV), 0.05, status.to(DEV).int(), 1, 5)

    P, C, pb, ptr = fcc_boxes(seed=5, n_boxes=6, reps=2, a=1.5496, jitter=0.02)
    N = len(P)
    batch = make_batch(P, np.full(N, 18, dtype=np.int64), np.ones(N, dtype=np.float32), C, pb, ptr)
    f = torch.randn(N, 3, generator=g) * torch.repeat_interleave(torch.tensor([0.001, 1.0, 0.01, 0.5, 0.002, 2.0]), N // 6)[:, None]
    batch.forces.copy_(f.to(DEV))
    start = torch.tensor([0, 0, 1, 0, 2, 0], dtype=torch.long, device=DEV).view(-1, 1)
    one = ConvergenceHook.from_fmax(0.05, source_status=0, target_status=1)
    two = ConvergenceHook(criteria=[{"key": "forces", "threshold": 0.05, "reduce_op": "norm"},
                                    {"key": "energy", "threshold": 1e30}], source_status=0, target_status=1)
    out = []
    for hook in (one, two):
        batch.status = start.clone()
        hook(DynamicsContext(batch=batch, model=None, workflow=None), None)
        out.append(batch.status.clone())
    assert torch.equal(out[0], out[1]) and out[0].view(-1).tolist() == [1, 0, 1, 0, 2, 0]


def test_joined_velocity_verlet_halves_equal_the_two_calls_in_a_row():
    """nvamd_vv_finalize_then_update against nvamd_vv_velocity_finalize followed by nvamd_vv_position_update with the
    same forces: bit for bit, with and without a system mask, on aligned arrays (four floats per lane) and on views
    that start off a 16-byte boundary (one float per lane), for atom counts around the lane boundaries."""
    from nvalchemi_amd import _lib

    g = torch.Generator().manual_seed(11)
    for N in (1, 2, 5, 255, 256, 1027):
        M = 4
        bidx = torch.sort(torch.randint(0, M, (N,), generator=g)).values.to(torch.int32).to(DEV)
        base = [torch.randn(N + 1, 3, generator=g).to(DEV) for _ in range(3)]
        masses = (torch.rand(N, generator=g) * 20 + 1).to(DEV)
        dt = (torch.rand(M, generator=g) * 0.1 + 0.01).to(DEV)
        for active in (None, torch.tensor([True, False, True, True], device=DEV)):
            for offset in (0, 1):  # (offset 1: the rows start 12 bytes into the allocation)
                P0, V0, F = (b[offset:offset + N] for b in base)
                Pa, Va = P0.clone(), V0.clone()
                Pb, Vb = P0.clone(), V0.clone()
                if offset:
                    hold = [torch.empty(N + 1, 3, device=DEV) for _ in range(4)]
                    Pa, Va, Pb, Vb = (h[1:] for h in hold)
                    Pa.copy_(P0); Va.copy_(V0); Pb.copy_(P0); Vb.copy_(V0)
                    assert Pa.data_ptr() % 16 != 0
                _lib.vv_velocity_finalize(Va, F, masses, dt, bidx, active)
                _lib.vv_position_update(Pa, Va, F, masses, dt, bidx, active)
                _lib.vv_finalize_then_update(Pb, Vb, F, masses, dt, bidx, active)
                assert torch.equal(Pa, Pb) and torch.equal(Va, Vb), (N, active is not None, offset)
                if active is not None and bool((bidx == 1).any()):
                    off = (bidx == 1)
                    assert torch.equal(Pb[off], P0[off]) and torch.equal(Vb[off], V0[off])


def test_runs_replayed_four_steps_at_a_time_equal_eager_ones():
    """``run`` replays four steps per graph where it may (NVE, no hook around the step boundary, no status), with the
    closing half kick of a step and the opening half kick and drift of the next in one launch: positions, velocities
    and forces after 3 to 23 steps equal those of eager steps bit for bit, whatever is left over after the last
    group of four; with a hook registered after the step, or a status on the batch, steps are replayed one at a
    time."""
    from nvalchemi_amd.dynamics import NVE, DynamicsStage
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=9, n_boxes=4, reps=3, a=3.7, jitter=0.08)
    n = len(P)
    V = np.random.default_rng(9).normal(0, 0.02, (n, 3)).astype(np.float32)
    sigma = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))

    def make():
        batch = make_batch(P, np.full(n, 29, dtype=np.int64), np.full(n, 63.546, dtype=np.float32), C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=sigma, cutoff=5.0)
        return batch, NVE(model, dt=1.0, hooks=model.make_neighbor_hooks())

    for n_steps in (3, 6, 7, 12, 23):
        out = []
        for replay in (False, True):
            batch, dyn = make()
            dyn.graph_replay = replay
            dyn.run(batch, n_steps=n_steps)
            torch.cuda.synchronize()
            assert dyn.step_count == n_steps
            if replay:
                # (a few eager steps while the hook settles its buffers, one step replayed alone, then up to four at a
                # time: what is left over after the groups of four is a group of two or three, or a single step)
                joined = dyn._graph_state.get("joined")
                assert not joined if n_steps <= 3 else (bool(joined) or n_steps < 12), n_steps
                if n_steps == 23:
                    assert 4 in joined and len(joined) >= 2
            out.append(batch)
        for name in ("positions", "velocities", "forces", "energy"):
            assert torch.equal(getattr(out[0], name), getattr(out[1], name)), (name, n_steps)
    # two runs in a row use the graphs of the first
    batch, dyn = make()
    dyn.run(batch, n_steps=9)
    first = dyn._graph_state["joined"][4]
    dyn.run(batch, n_steps=9)
    eager_batch, eager = make()
    eager.graph_replay = False
    eager.run(eager_batch, n_steps=18)
    assert dyn._graph_state["joined"][4] is first and torch.equal(batch.positions, eager_batch.positions)

    class Watch:
        frequency = 1
        graph_safe = True
        stage = DynamicsStage.AFTER_STEP

        def __call__(self, ctx, stage):
            pass

    batch, dyn = make()
    dyn.register_hook(Watch())
    dyn.run(batch, n_steps=12)
    assert dyn._graph_state["graph"] is not None and not dyn._graph_state.get("joined")
    batch, dyn = make()
    batch.status = torch.zeros(batch.num_graphs, 1, dtype=torch.long, device=DEV)
    dyn.run(batch, n_steps=12)
    assert dyn._graph_state["graph"] is not None and not dyn._graph_state.get("joined")
