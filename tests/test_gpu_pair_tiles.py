"""GPU tests of the pair kernel that walks the tiles of the neighbor search again (nvamd_nl_build_tiles,
nvamd_lj_energy_forces_tiles): systems too large for the pair kernel to stage whole.

What is checked: that the build's extra outputs describe its own search (every listed pair's tile index names
the listed neighbor; the units' rows are the atoms, once each); that the pair results are those of the entry
point that gathers neighbors from memory, which the other tests hold against the oracle (bit for bit where
both sum in the same order: diagonal cells, rows of up to 384 slots; to the float32 bar of 1e-5 relative /
1e-6 absolute elsewhere), on cubic and triclinic cells, several systems, cells too narrow for derived images,
systems too dense for one tile; one case directly against the oracle; and the way through the hook and the
model, including that tiles of other positions are not used.
"""

import numpy as np
import pytest
import torch

import oracle
from _systems import periodic_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def build_with_tiles(P, C, pb, ptr, rc, K, sort_path=None):
    from nvalchemi_amd import _lib

    N, B = len(P), len(C)
    pos, cell, pbc = T(P, torch.float32), T(C, torch.float32), T(pb)
    tptr = T(ptr, torch.int32)
    bidx = torch.repeat_interleave(torch.arange(B, dtype=torch.int32, device=DEV), (tptr[1:] - tptr[:-1]).long())
    nm = torch.full((N, K), N, dtype=torch.int32, device=DEV)
    nn = torch.zeros(N, dtype=torch.int32, device=DEV)
    sh = torch.zeros((N, K, 3), dtype=torch.int32, device=DEV)
    tiles = (torch.full((N, K), -1, dtype=torch.int16, device=DEV), torch.empty(N, 4, dtype=torch.float32, device=DEV),
             torch.full((_lib.nl_tile_records(N, B), _lib.NL_TILE_RECORD_INTS), -7, dtype=torch.int32, device=DEV),
             torch.zeros(1, dtype=torch.int32, device=DEV))
    _lib.nl_build(pos, cell, pbc, tptr, bidx, None, rc, K, False, 1, nm, nn, sh, sort_path=sort_path, pair_tiles=tiles)
    order = torch.empty(N, dtype=torch.int32, device=DEV)
    _lib.nl_atom_order(bidx, B, order)
    torch.cuda.synchronize()
    assert int(nn.max()) < K, "rows too short for this case"
    return dict(pos=pos, cell=cell, bidx=bidx, nm=nm, nn=nn, sh=sh, tiles=tiles, order=order, N=N, B=B, K=K, rc=rc)


def pair(b, eps, sig, tiles, virial=False):
    from nvalchemi_amd import _lib

    e = torch.empty(b["N"], dtype=torch.float32, device=DEV)
    f = torch.empty((b["N"], 3), dtype=torch.float32, device=DEV)
    w = torch.empty((b["B"], 9), dtype=torch.float32, device=DEV) if virial else None
    es = torch.empty(b["B"], dtype=torch.float32, device=DEV)
    _lib.lj_energy_forces(b["pos"], b["cell"], b["nm"], b["sh"], b["nn"], b["bidx"], b["N"], eps, sig, b["rc"], 0.0, False,
                          e, f, w, es, row_order=b["order"], neighbor_list_cutoff=b["rc"],
                          pair_tiles=b["tiles"] if tiles else None)
    torch.cuda.synchronize()
    return e, f, w, es


def close(got, want):
    want = want.double()
    return bool(((got.double() - want).abs() <= 1e-6 + 1e-5 * want.abs()).all())


def unit_table(b):
    """(first row, rows, system, atoms in the tile) and the per-cell (first slot, offset) tables of the units."""
    index, ordered, records, count = b["tiles"]
    nu = int(count.item())
    rec = records[:nu].view(nu, -1, 2)
    return nu, rec[:, 0, 0], rec[:, 0, 1], rec[:, 1, 0], rec[:, 1, 1], rec[:, 2:, 0], rec[:, 2:, 1]


@pytest.mark.parametrize("sort_path", [1, 2], ids=["per_system_sort", "global_sort"])
def test_the_builds_tiles_describe_its_own_search(sort_path):
    """The units' rows are every slot of the cell order once; the atom in slot k of that order is ordered_positions'
    fourth word and its first three are that atom's coordinates; and for every listed pair, the atom that stands at
    the pair's tile index in the tile of the row's unit (laid out by the unit's record) is the listed neighbor."""
    P, C, pb, ptr = periodic_batch(seed=11, n_systems=3, n_lo=5000, n_hi=7000, density=0.1)
    b = build_with_tiles(P, C, pb, ptr, 5.0, 96, sort_path=sort_path)
    N, K = b["N"], b["K"]
    index, ordered, records, count = b["tiles"]
    nu, first, rows, system, tile_n, cell_start, cell_off = unit_table(b)
    assert 0 < nu <= records.shape[0]
    # rows: a partition of the slots, units inside their systems
    keep = rows > 0
    by_first = torch.argsort(first[keep])
    f_sorted, r_sorted = first[keep][by_first], rows[keep][by_first]
    assert int(f_sorted[0]) == 0 and int((f_sorted + r_sorted)[-1]) == N
    assert bool((f_sorted[1:] == (f_sorted + r_sorted)[:-1]).all())
    unit_ids = torch.arange(nu, device=DEV)[keep][by_first]
    unit_of_slot = torch.repeat_interleave(unit_ids, r_sorted.long())
    # the cell order
    atom_of_slot = ordered[:, 3].contiguous().view(torch.int32)
    assert bool((atom_of_slot == b["order"]).all())
    assert torch.equal(ordered[:, :3], b["pos"][atom_of_slot.long()])
    assert bool((b["bidx"][atom_of_slot.long()] == system[unit_of_slot]).all())
    # every unit of this case has a tile, no larger than the limit
    assert bool((tile_n[keep] > 0).all()) and int(tile_n.max()) <= 1088
    # the pairs
    slot_of_atom = torch.empty(N, dtype=torch.long, device=DEV)
    slot_of_atom[atom_of_slot.long()] = torch.arange(N, device=DEV)
    i, s = torch.nonzero(torch.arange(K, device=DEV)[None, :] < b["nn"][:, None], as_tuple=True)
    k = index[i, s].long() & 0xffff
    u = unit_of_slot[slot_of_atom[i]]
    assert bool((k < tile_n[u]).all())
    found = torch.empty_like(k)
    for lo in range(0, len(k), 1 << 20):  # (in pieces: a 64-wide comparison per pair)
        kk, uu = k[lo:lo + (1 << 20)], u[lo:lo + (1 << 20)]
        c = (cell_off[uu] <= kk[:, None]).sum(1) - 1
        src = cell_start[uu, c] + kk - cell_off[uu, c]
        found[lo:lo + (1 << 20)] = atom_of_slot[src.long()]
    assert bool((found == b["nm"][i, s]).all())


@pytest.mark.parametrize("virial", [False, True])
def test_cubic_boxes_bit_for_bit_with_the_gathering_kernel(virial):
    P, C, pb, ptr = periodic_batch(seed=12, n_systems=2, n_lo=20000, n_hi=30000, density=0.1)
    b = build_with_tiles(P, C, pb, ptr, 6.0, 160)
    e0, f0, w0, s0 = pair(b, 0.01, 1.5, tiles=False, virial=virial)
    e1, f1, w1, s1 = pair(b, 0.01, 1.5, tiles=True, virial=virial)
    assert torch.equal(e0, e1) and torch.equal(f0, f1)
    assert close(s1, s0)
    if virial:
        scale = w0.abs().max()
        assert bool(((w1 - w0).abs() <= 1e-5 * scale).all())


def test_one_system_against_the_oracle():
    P, C, pb, ptr = periodic_batch(seed=13, n_systems=1, n_lo=6000, n_hi=6000, density=0.08)
    rc, eps, sig = 5.0, 0.01, 2.0
    b = build_with_tiles(P, C, pb, ptr, rc, 96)
    e1, f1, _, s1 = pair(b, eps, sig, tiles=True)
    bi = oracle.batch_idx_from_ptr(ptr)
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc, 96)
    ref = oracle.lj_matrix(P, C, nm, sh, nn, bi, len(P), eps, sig, rc)
    assert close(e1.cpu(), torch.from_numpy(ref["atomic_energies"]))
    # (random positions: a few pairs nearly touch, their forces are huge and cancel in part against others)
    want = torch.from_numpy(ref["forces"]).double()
    tol = 1e-6 + 1e-5 * want.abs().amax(1, keepdim=True)
    assert bool(((f1.cpu().double() - want).abs() <= tol).all())
    assert close(s1.cpu(), torch.from_numpy(ref["energy"]))


def test_triclinic_systems_take_the_general_image():
    """Sheared cells, wide enough for derived images: the images come from the inverse cell (and the sums are taken
    in another order than in the gathering kernel, four entries a lane there, eight here)."""
    P, C, pb, ptr = periodic_batch(seed=14, n_systems=3, n_lo=5000, n_hi=9000, density=0.08, triclinic=True, spread=0.3)
    b = build_with_tiles(P, C, pb, ptr, 5.0, 160)
    e0, f0, w0, s0 = pair(b, 0.01, 2.0, tiles=False, virial=True)
    e1, f1, w1, s1 = pair(b, 0.01, 2.0, tiles=True, virial=True)
    assert close(e1, e0) and close(s1, s0)
    tol = 1e-6 + 1e-5 * f0.double().abs().amax(1, keepdim=True)
    assert bool(((f1.double() - f0.double()).abs() <= tol).all())
    assert bool(((w1 - w0).abs() <= 1e-5 * w0.abs().max()).all())
    assert float((e1 == e0).float().mean()) > 0.999


def test_a_cell_too_narrow_for_derived_images_reads_its_shifts():
    """One system in a cell thinner than twice the cutoff along x (its shifts have to be read) beside one in a cube."""
    rng = np.random.default_rng(15)
    cells = np.stack([np.diag([5.0, 40.0, 400.0]), np.eye(3) * 40.0]).astype(np.float32)
    counts = [8000, 6400]
    P = np.concatenate([(rng.uniform(0, 1, (n, 3)) @ c.astype(np.float64)).astype(np.float32) for n, c in zip(counts, cells)])
    ptr = np.array([0, counts[0], sum(counts)], dtype=np.int32)
    pb = np.ones((2, 3), dtype=bool)
    b = build_with_tiles(P, cells, pb, ptr, 3.0, 48)
    e0, f0, _, s0 = pair(b, 0.01, 1.2, tiles=False)
    e1, f1, _, s1 = pair(b, 0.01, 1.2, tiles=True)
    assert bool((b["sh"][:8000].abs().amax((1, 2)) > 0).any())  # (pairs through the thin direction are there)
    assert close(e1, e0) and close(s1, s0)
    tol = 1e-6 + 1e-5 * f0.double().abs().amax(1, keepdim=True)
    assert bool(((f1.double() - f0.double()).abs() <= tol).all())
    assert torch.equal(e0[8000:], e1[8000:]) and torch.equal(f0[8000:], f1[8000:])


def test_units_whose_stencil_is_more_than_one_tile_gather_from_memory():
    """Dense enough that the 27 cells around a cell hold more atoms than a tile takes: the records say "no tile"
    and the rows of those units find their neighbors in memory."""
    P, C, pb, ptr = periodic_batch(seed=16, n_systems=1, n_lo=9000, n_hi=9000, density=0.35)
    b = build_with_tiles(P, C, pb, ptr, 6.0, 448)
    nu, first, rows, system, tile_n, _, _ = unit_table(b)
    assert bool(((tile_n < 0) & (rows > 0)).any())
    e0, f0, _, s0 = pair(b, 0.001, 1.0, tiles=False)
    e1, f1, _, s1 = pair(b, 0.001, 1.0, tiles=True)
    assert close(e1, e0) and close(s1, s0)
    tol = 1e-6 + 1e-5 * f0.double().abs().amax(1, keepdim=True)
    assert bool(((f1.double() - f0.double()).abs() <= tol).all())


def test_what_the_tile_entries_refuse():
    from nvalchemi_amd import _lib

    P, C, pb, ptr = periodic_batch(seed=17, n_systems=1, n_lo=5000, n_hi=5000, density=0.1)
    with pytest.raises(Exception, match="multiple of 8"):
        build_with_tiles(P, C, pb, ptr, 5.0, 100)
    b = build_with_tiles(P, C, pb, ptr, 5.0, 96)
    index, ordered, records, count = b["tiles"]
    flags = torch.ones(1, dtype=torch.bool, device=DEV)
    with pytest.raises(ValueError, match="every system"):
        _lib.nl_build(b["pos"], b["cell"], T(pb), T(ptr, torch.int32), b["bidx"], flags, 5.0, 96, False, 1, b["nm"], b["nn"],
                      b["sh"], pair_tiles=b["tiles"])
    with pytest.raises(ValueError, match="full list"):
        _lib.nl_build(b["pos"], b["cell"], T(pb), T(ptr, torch.int32), b["bidx"], None, 5.0, 96, True, 1, b["nm"], b["nn"],
                      b["sh"], pair_tiles=b["tiles"])
    with pytest.raises(Exception, match="tile_records"):
        _lib.nl_build(b["pos"], b["cell"], T(pb), T(ptr, torch.int32), b["bidx"], None, 5.0, 96, False, 1, b["nm"], b["nn"],
                      b["sh"], pair_tiles=(index, ordered, records[:10], count))


def test_hook_and_model_use_the_tiles_of_the_positions_in_hand_only():
    """Through NeighborListHook and the model: a batch of systems of more than 4096 atoms gets its tiles published
    and the model's results are those of a model that is kept from seeing them; after the positions have been
    written the stale tiles are left alone."""
    import sys
    sys.path.insert(0, ".")
    import bench
    from nvalchemi_amd.hooks._context import HookContext
    from nvalchemi_amd.models import LennardJonesModelWrapper

    g = torch.Generator().manual_seed(5)
    L = (6000 / 0.1) ** (1 / 3)
    systems = [(torch.rand(6000, 3, generator=g) * L, torch.eye(3) * L) for _ in range(2)]
    batch = bench._batch_of(systems, torch.device(DEV))
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=1.5, cutoff=6.0)
    hook = model.make_neighbor_hooks()[0]
    ctx = HookContext(batch=batch, model=model, workflow=None)
    hook(ctx, hook.stage)
    hook(ctx, hook.stage)  # (the first call sizes the rows; from the second on the tiles are those of the rows in use)
    tiles = batch._neighbor_pair_tiles
    assert tiles is not None and tiles[4] == batch.positions.data_ptr()
    out1 = model(batch)
    e1, f1 = out1["energy"].clone(), out1["forces"].clone()
    object.__setattr__(batch, "_neighbor_pair_tiles", None)
    out0 = model(batch)
    assert torch.equal(out0["forces"], f1) and close(e1, out0["energy"])
    # the positions move: the matrix still holds every pair within the cutoff (nothing moves further than 1e-3), the
    # tiles' coordinates are the old ones
    object.__setattr__(batch, "_neighbor_pair_tiles", tiles)
    batch.positions.add_(1e-3 * torch.rand(batch.positions.shape, generator=g).to(DEV))
    out2 = model(batch)
    f2 = out2["forces"].clone()
    object.__setattr__(batch, "_neighbor_pair_tiles", None)
    out3 = model(batch)
    assert torch.equal(out3["forces"], f2)
    assert not torch.equal(f2, f1)
