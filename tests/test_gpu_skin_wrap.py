"""GPU parity of the Verlet-skin displacement test, the selective rebuild driven by it, and the
periodic wrap (all through the C ABI) against the CPU oracle.

Bars: rebuild flags and refreshed reference positions bit-exact; wrapped positions bit-exact (both
sides evaluate the same double-precision expression and round once); neighbor data after a
skin-driven selective rebuild bit-exact as sorted (i, j, shift) sets against a full build at
``cutoff + skin`` on the positions each system had when it was last flagged; trajectories with and
without a skin within 1e-5 relative / 1e-6 absolute.
"""

import numpy as np
import pytest
import torch

import oracle
from _systems import fcc_boxes, periodic_batch
from test_gpu_dynamics import close, make_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


@pytest.mark.parametrize("with_cell,pbc", [(False, None), (True, [1, 1, 1]), (True, [1, 0, 1]), (True, [0, 0, 0])])
@pytest.mark.parametrize("update", [False, True])
def test_rebuild_check_matches_oracle(with_cell, pbc, update):
    from nvalchemi_amd.dynamics._ops.neighbor_list_rebuild import batch_neighbor_list_rebuild_inplace

    P, C, pb, ptr = periodic_batch(seed=5, n_systems=40, n_lo=1, n_hi=60, density=0.05, triclinic=True, spread=0.3)
    rng = np.random.default_rng(6)
    bi = oracle.batch_idx_from_ptr(ptr)
    B = len(ptr) - 1
    # small thermal motion everywhere, a few atoms beyond the threshold, a few moved by whole
    # lattice vectors (no displacement where the axis is periodic)
    cur = P + rng.normal(0, 0.02, P.shape).astype(np.float32)
    movers = rng.choice(len(P), 12, replace=False)
    cur[movers[:6]] += rng.normal(0, 0.4, (6, 3)).astype(np.float32)
    for i in movers[6:]:
        cur[i] += C[bi[i]][rng.integers(0, 3)] * rng.choice([-1, 1])
    cell = C if with_cell else None
    pbv = None if pbc is None else np.broadcast_to(np.array(pbc, bool), (B, 3)).copy()
    flags_ref, ref_after = oracle.rebuild_check(P, cur, bi, B, 0.25, update, cell, pbv)
    assert 0 < flags_ref.sum() < B
    ref_t = _dev(P)
    flags_t = torch.ones(B, dtype=torch.bool, device=DEV)  # stale content must be cleared
    batch_neighbor_list_rebuild_inplace(
        reference_positions=ref_t, current_positions=_dev(cur), batch_idx=_dev(bi), rebuild_flags=flags_t,
        skin_distance_threshold=0.25, update_reference_positions=update,
        cell=None if cell is None else _dev(cell), cell_inv=None, pbc=None if pbv is None else _dev(pbv))
    torch.cuda.synchronize()
    assert np.array_equal(flags_t.cpu().numpy(), flags_ref)
    assert np.array_equal(ref_t.cpu().numpy(), ref_after)


def test_rebuild_check_shape_mismatch_flags_everything():
    from nvalchemi_amd.dynamics._ops.neighbor_list_rebuild import batch_neighbor_list_rebuild_inplace

    flags = torch.zeros(3, dtype=torch.bool, device=DEV)
    batch_neighbor_list_rebuild_inplace(torch.zeros(4, 3, device=DEV), torch.zeros(5, 3, device=DEV),
                                        torch.zeros(5, dtype=torch.int32, device=DEV), flags, 0.5)
    assert bool(flags.all())


@pytest.mark.parametrize("pbc", [[1, 1, 1], [1, 1, 0], [0, 1, 0], [0, 0, 0]])
def test_wrap_matches_oracle(pbc):
    from nvalchemi_amd.hooks import wrap_positions_into_cell

    P, C, pb, ptr = periodic_batch(seed=9, n_systems=30, n_lo=1, n_hi=80, density=0.05, triclinic=True, spread=3.0)
    B = len(ptr) - 1
    pbv = np.broadcast_to(np.array(pbc, bool), (B, 3)).copy()
    pbv[::7] = [True, False, True]  # mixed flags inside one batch
    bi = oracle.batch_idx_from_ptr(ptr)
    expect = oracle.wrap_positions(P, C, pbv, bi)
    pos = _dev(P)
    out = wrap_positions_into_cell(pos, _dev(C), _dev(pbv), _dev(bi))
    assert out is pos
    assert np.array_equal(pos.cpu().numpy(), expect)
    # wrapping what is already wrapped moves nothing by more than rounding
    again = oracle.wrap_positions(expect, C, pbv, bi)
    wrap_positions_into_cell(pos, _dev(C), _dev(pbv), _dev(bi))
    assert np.array_equal(pos.cpu().numpy(), again)


def _line_batch():
    from nvalchemi_amd.data import AtomicData, Batch

    pos = torch.tensor([[0.0, 0.0, 0.0], [1.5, 0.0, 0.0], [5.0, 0.0, 0.0]])
    return Batch.from_data_list([AtomicData(pos, torch.tensor([1, 1, 1]))], device=DEV)


def _hook(skin, fmt="matrix"):
    from nvalchemi_amd.hooks import HookContext, NeighborListHook
    from nvalchemi_amd.models.base import NeighborConfig, NeighborListFormat

    cfg = NeighborConfig(cutoff=2.5, format=NeighborListFormat.COO if fmt == "coo" else NeighborListFormat.MATRIX)
    return NeighborListHook(cfg, skin=skin), HookContext


def _ctx(HookContext, batch):
    return HookContext(batch=batch)


def test_hook_skin_state_follows_the_reference_protocol():
    """Restates test/hooks/test_neighbor_list_hook.py:825-893."""
    hook, HookContext = _hook(0.5)
    assert hook._ref_positions is None
    batch = _line_batch()
    hook(_ctx(HookContext, batch), None)
    assert hook._ref_positions is not None and hook._ref_positions.shape == (3, 3)
    nn_first = batch.num_neighbors.clone()
    hook(_ctx(HookContext, batch), None)
    assert torch.equal(nn_first, batch.num_neighbors)
    assert not bool(hook._rebuild_flags.any())  # nothing moved: nothing rebuilt
    batch.positions[2, 0] = 2.0  # 0.5 from atom 1: a displacement of 3 > skin / 2
    hook(_ctx(HookContext, batch), None)
    assert bool(hook._rebuild_flags.all())
    nm, nn = batch.neighbor_matrix.cpu(), batch.num_neighbors.cpu()
    assert 2 in nm[1, : nn[1]].tolist()
    hook0, _ = _hook(0.0)
    hook0(_ctx(HookContext, _line_batch()), None)
    assert hook0._ref_positions is None


def test_hook_skin_rebuild_leaves_no_stale_edges():
    """Restates test/hooks/test_neighbor_list_hook.py:1051-1090 (COO format, skin 1.0)."""
    hook, HookContext = _hook(1.0, "coo")
    batch = _line_batch()
    hook(_ctx(HookContext, batch), None)
    before = {tuple(r) for r in batch.neighbor_list.cpu().tolist()}
    assert (0, 1) in before and (1, 0) in before
    batch.positions[1, 0] = 4.0  # 4.0 from atom 0 (> cutoff + skin), 1.0 from atom 2
    hook(_ctx(HookContext, batch), None)
    after = {tuple(r) for r in batch.neighbor_list.cpu().tolist()}
    assert (0, 1) not in after and (1, 0) not in after
    assert (1, 2) in after and (2, 1) in after
    counts = torch.bincount(batch.neighbor_list[:, 0].cpu(), minlength=3)
    assert torch.equal(counts, hook._num_neighbors.cpu().to(counts.dtype))


def test_selective_rebuild_keeps_old_rows_and_rebuilds_flagged_systems_exactly():
    from nvalchemi_amd.hooks import HookContext, NeighborListHook
    from nvalchemi_amd.models.base import NeighborConfig, NeighborListFormat

    P, C, pb, ptr = fcc_boxes(seed=2, n_boxes=4, reps=3, a=3.6)
    N = len(P)
    rc, skin = 4.0, 0.6
    batch = make_batch(P, np.full(N, 29, np.int64), np.ones(N, np.float32), C, pb, ptr)
    hook = NeighborListHook(NeighborConfig(cutoff=rc, format=NeighborListFormat.MATRIX), skin=skin)
    hook(HookContext(batch=batch), None)
    # move every atom a little (below skin / 2), and one atom of systems 1 and 3 a lot
    rng = np.random.default_rng(4)
    P2 = P + rng.normal(0, 0.03, P.shape).astype(np.float32)
    P2[ptr[1] + 5] += np.array([0.5, 0.2, 0.0], np.float32)
    P2[ptr[3] + 7] += np.array([0.0, 0.0, -0.45], np.float32)
    batch.positions.copy_(torch.from_numpy(P2))
    hook(HookContext(batch=batch), None)
    assert hook._rebuild_flags.cpu().tolist() == [False, True, False, True]
    # what each system's rows must hold: a full build at cutoff + skin on the positions of its last build
    P_last = P.copy()
    for s in (1, 3):
        P_last[ptr[s]:ptr[s + 1]] = P2[ptr[s]:ptr[s + 1]]
    ref = oracle.nl_brute(P_last, C, pb, ptr, rc + skin)
    got = oracle.matrix_to_edges(batch.neighbor_matrix.cpu().numpy(), batch.num_neighbors.cpu().numpy(),
                                 batch.neighbor_matrix_shifts.cpu().numpy())
    assert np.array_equal(got, ref)
    assert np.array_equal(hook._ref_positions.cpu().numpy(), P_last)


def test_nve_trajectory_with_a_skin_equals_the_one_without():
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=3, reps=3, a=3.6)
    N = len(P)
    rng = np.random.default_rng(1)
    M = np.full(N, 63.546, dtype=np.float32)
    V = rng.normal(0, 0.03, (N, 3)).astype(np.float32)
    Z = np.full(N, 29, dtype=np.int64)
    sig = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))
    out = {}
    rebuilds = 0
    for skin in (0.0, 0.5):
        batch = make_batch(P, Z, M, C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=sig, cutoff=4.5)
        hooks = model.make_neighbor_hooks()
        for h in hooks:
            h.skin = skin
        dyn = NVE(model, dt=2.0, hooks=hooks)
        for _ in range(150):
            dyn.run(batch, n_steps=1)
            if skin > 0 and bool(hooks[0]._rebuild_flags.any()):
                rebuilds += 1
        out[skin] = batch
    assert 0 < rebuilds < 150  # the skin did skip builds, and did trigger some
    for key in ("positions", "velocities", "forces", "energy"):
        close(getattr(out[0.5], key), getattr(out[0.0], key).cpu().numpy(), key)


def test_wrap_hook_in_a_periodic_run_changes_nothing_physical():
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.dynamics.base import DynamicsStage
    from nvalchemi_amd.hooks import WrapPeriodicHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=2, reps=3, a=3.6)
    N = len(P)
    M = np.full(N, 63.546, dtype=np.float32)
    V = np.tile(np.array([[0.4, -0.3, 0.2]], np.float32), (N, 1))  # a drift that carries atoms out of the box
    V += np.random.default_rng(2).normal(0, 0.01, (N, 3)).astype(np.float32)
    Z = np.full(N, 29, dtype=np.int64)
    sig = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))
    res = {}
    for wrap in (False, True):
        batch = make_batch(P, Z, M, C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=sig, cutoff=4.5)
        hooks = model.make_neighbor_hooks()
        if wrap:
            hooks.append(WrapPeriodicHook(frequency=5, stage=DynamicsStage.AFTER_POST_UPDATE))
        NVE(model, dt=2.0, hooks=hooks).run(batch, n_steps=120)
        res[wrap] = batch
    frac = res[True].positions.cpu().numpy().astype(np.float64) / 10.8
    assert frac.min() > -0.06 and frac.max() < 1.06          # wrapped run stays in the box (5 steps of drift at most)
    assert np.abs(res[False].positions.cpu().numpy() / 10.8).max() > 1.5  # the other one left it
    # Same physics, but not the same roundings: the two runs hold different absolute coordinates
    # in float32, so they agree to what 120 steps make of one-ulp differences, not to 1e-5.
    for key, tol in (("forces", 2e-4), ("velocities", 2e-5)):
        a = getattr(res[True], key).cpu().numpy().astype(np.float64)
        b = getattr(res[False], key).cpu().numpy().astype(np.float64)
        assert np.abs(a - b).max() < tol, (key, np.abs(a - b).max())
    assert abs(float(res[True].energy.sum() - res[False].energy.sum())) < 1e-4 * abs(float(res[False].energy.sum()))
    d = (res[True].positions - res[False].positions).cpu().numpy().astype(np.float64) / 10.8
    assert np.abs(d - np.round(d)).max() < 1e-4


def test_skin_and_wrap_together_on_cells_whose_shifts_are_read():
    """Cells narrower than twice the search radius (the pair kernel reads the stored shifts there) with a
    Verlet skin AND the wrap hook: an atom that the wrap moves by a lattice vector between two builds
    must make its system's list be built afresh, or the kept rows would pair its new coordinates with the
    shifts of the old ones.  The run with the wrap must be the run without it, up to lattice vectors."""
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.dynamics.base import DynamicsStage
    from nvalchemi_amd.hooks import WrapPeriodicHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=3, n_boxes=3, reps=2, a=3.6)  # 7.2 wide: less than 2 (4.5 + 0.5)
    N = len(P)
    M = np.full(N, 63.546, dtype=np.float32)
    V = np.tile(np.array([[0.35, -0.25, 0.15]], np.float32), (N, 1))  # a drift that carries atoms across the faces
    V += np.random.default_rng(5).normal(0, 0.01, (N, 3)).astype(np.float32)
    Z = np.full(N, 29, dtype=np.int64)
    sig = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))
    res, kept = {}, 0
    for wrap in (False, True):
        batch = make_batch(P, Z, M, C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=sig, cutoff=4.5)
        hooks = model.make_neighbor_hooks()
        for h in hooks:
            h.skin = 0.5
        if wrap:
            hooks.append(WrapPeriodicHook(frequency=1, stage=DynamicsStage.AFTER_POST_UPDATE))
        dyn = NVE(model, dt=2.0, hooks=hooks)
        for _ in range(100):
            dyn.run(batch, n_steps=1)
            if wrap and not bool(hooks[0]._rebuild_flags.all()):
                kept += 1
        res[wrap] = batch
    assert kept > 20  # the skin did keep lists in the wrapped run
    assert np.abs(res[False].positions.cpu().numpy() / 7.2).max() > 1.3  # atoms did leave the box
    frac = res[True].positions.cpu().numpy().astype(np.float64) / 7.2
    assert frac.min() > -0.02 and frac.max() < 1.02
    for key, tol in (("forces", 2e-4), ("velocities", 2e-5)):
        a = getattr(res[True], key).cpu().numpy().astype(np.float64)
        b = getattr(res[False], key).cpu().numpy().astype(np.float64)
        assert np.abs(a - b).max() < tol, (key, np.abs(a - b).max())
    d = (res[True].positions - res[False].positions).cpu().numpy().astype(np.float64) / 7.2
    assert np.abs(d - np.round(d)).max() < 1e-4


def test_min_image_skin_keeps_lists_through_wraps_on_cells_whose_shifts_are_derived():
    """Cells wider than twice the search radius (the pair kernel derives the shifts from the positions there)
    with a Verlet skin, the wrap hook and ``min_image_skin=True``: a wrap is no displacement, so the lists are
    kept through it (far fewer rebuilds than with the plain displacement), and the run is still the run without
    the wrap, up to lattice vectors."""
    from nvalchemi_amd.dynamics import NVE
    from nvalchemi_amd.dynamics.base import DynamicsStage
    from nvalchemi_amd.hooks import WrapPeriodicHook
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P, C, pb, ptr = fcc_boxes(seed=4, n_boxes=3, reps=4, a=3.6)  # 14.4 wide: more than 2 (4.5 + 0.5)
    N = len(P)
    M = np.full(N, 63.546, dtype=np.float32)
    V = np.tile(np.array([[0.35, -0.25, 0.15]], np.float32), (N, 1))  # a drift that carries atoms across the faces
    V += np.random.default_rng(5).normal(0, 0.01, (N, 3)).astype(np.float32)
    Z = np.full(N, 29, dtype=np.int64)
    sig = float((3.6 / np.sqrt(2)) / 2 ** (1 / 6))
    res, rebuilt = {}, {}
    for mode in ("no wrap", "plain", "min image"):
        batch = make_batch(P, Z, M, C, pb, ptr, V)
        model = LennardJonesModelWrapper(epsilon=0.01, sigma=sig, cutoff=4.5)
        hooks = model.make_neighbor_hooks()
        for h in hooks:
            h.skin = 0.5
            h.min_image_skin = mode == "min image"
        if mode != "no wrap":
            hooks.append(WrapPeriodicHook(frequency=1, stage=DynamicsStage.AFTER_POST_UPDATE))
        dyn = NVE(model, dt=2.0, hooks=hooks)
        dyn.graph_replay = False
        n = 0
        for _ in range(100):
            dyn.run(batch, n_steps=1)
            n += int(hooks[0]._rebuild_flags.sum())
        res[mode], rebuilt[mode] = batch, n
    assert rebuilt["min image"] <= rebuilt["no wrap"] + 3 and rebuilt["plain"] > rebuilt["min image"] + 30
    assert np.abs(res["no wrap"].positions.cpu().numpy() / 14.4).max() > 1.1  # atoms did leave the box
    for mode in ("plain", "min image"):
        for key, tol in (("forces", 2e-4), ("velocities", 2e-5)):
            a = getattr(res[mode], key).cpu().numpy().astype(np.float64)
            b = getattr(res["no wrap"], key).cpu().numpy().astype(np.float64)
            assert np.abs(a - b).max() < tol, (mode, key, np.abs(a - b).max())
        d = (res[mode].positions - res["no wrap"].positions).cpu().numpy().astype(np.float64) / 14.4
        assert np.abs(d - np.round(d)).max() < 1e-4
