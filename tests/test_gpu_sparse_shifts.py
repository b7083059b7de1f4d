"""GPU tests of neighbor builds that leave zero shifts over zeros unwritten (``shift_groups`` of
nvamd_nl_build_extras).

The bar: after every build of a sequence on persistent buffers, ``num_neighbors`` and every row's set of
(neighbor, shift) pairs are exactly those of a build into fresh buffers from the same positions (the order of a
row's entries follows the order of the atoms inside their cells, which no two builds promise to share), and every
slot beyond a row's count holds the padding: the fill value and a zero shift.  The sequences move atoms through the faces of their cells, so that rows gain and lose shifted pairs,
grow and shrink; they cover full and half lists, both sorting paths, rows of more than 32 groups of one slot,
systems built selectively (rebuild flags), stencils of more than one tile, and the reset that the contract asks
for after something else has written the buffers.
"""

import numpy as np
import pytest
import torch

from _systems import periodic_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


class Buffers:
    def __init__(self, N, K):
        self.nm = torch.full((N, K), N, dtype=torch.int32, device=DEV)
        self.nn = torch.zeros(N, dtype=torch.int32, device=DEV)
        self.sh = torch.zeros((N, K, 3), dtype=torch.int32, device=DEV)
        self.groups = torch.zeros(N, dtype=torch.int32, device=DEV)


def build(pos, cell, pbc, ptr, bidx, rc, K, half, out, sparse, flags=None, sort_path=None):
    from nvalchemi_amd import _lib

    _lib.nl_build(pos, cell, pbc, ptr, bidx, flags, rc, K, half, 0 if sparse else 1, out.nm, out.nn, out.sh,
                  sort_path=sort_path, shift_groups=out.groups if sparse else None)


def fresh_build(pos, cell, pbc, ptr, bidx, rc, K, half, sort_path=None):
    out = Buffers(pos.shape[0], K)
    build(pos, cell, pbc, ptr, bidx, rc, K, half, out, sparse=False, sort_path=sort_path)
    return out


def rows_as_sets(b, N):
    """Per row, the sorted keys of its (neighbor, shift) entries; unused slots sort last."""
    K = b.nm.shape[1]
    used = torch.arange(K, device=DEV)[None, :] < b.nn[:, None]
    s = b.sh.long() + 512
    key = ((b.nm.long() * 1024 + s[..., 0]) * 1024 + s[..., 1]) * 1024 + s[..., 2]
    key = torch.where(used, key, torch.full_like(key, 1 << 62))
    return torch.sort(key, dim=1).values


def same_lists(kept, want, N):
    K = kept.nm.shape[1]
    unused = torch.arange(K, device=DEV)[None, :] >= kept.nn[:, None]
    return (torch.equal(kept.nn, want.nn) and torch.equal(rows_as_sets(kept, N), rows_as_sets(want, N))
            and bool((kept.nm[unused] == N).all()) and bool((kept.sh[unused] == 0).all()))


def system(seed, n_systems, n_lo, n_hi, density, triclinic=False):
    P, C, pb, ptr = periodic_batch(seed=seed, n_systems=n_systems, n_lo=n_lo, n_hi=n_hi, density=density, triclinic=triclinic)
    tptr = T(ptr, torch.int32)
    B = len(C)
    bidx = torch.repeat_interleave(torch.arange(B, dtype=torch.int32, device=DEV), (tptr[1:] - tptr[:-1]).long())
    return T(P, torch.float32), T(C, torch.float32), T(pb), tptr, bidx


def drift(pos, cell, bidx, g, step):
    """Every atom moves by up to ``step``; then all are wrapped back into their cells, so that atoms change sides."""
    from nvalchemi_amd import _lib

    pos.add_(step * (torch.rand(pos.shape, generator=g, device="cpu").to(DEV) - 0.3))
    frac = torch.linalg.solve(cell[bidx.long()].transpose(1, 2).double(), pos.double().unsqueeze(-1)).squeeze(-1)
    pos.copy_((torch.bmm((frac - torch.floor(frac)).unsqueeze(1), cell[bidx.long()].double()).squeeze(1)).float())


CASES = [
    ("full_small_boxes", dict(seed=21, n_systems=6, n_lo=300, n_hi=900, density=0.1), 5.0, 96, False, None),
    ("half_small_boxes", dict(seed=22, n_systems=6, n_lo=300, n_hi=900, density=0.1), 5.0, 112, True, None),
    ("triclinic", dict(seed=23, n_systems=5, n_lo=200, n_hi=700, density=0.08, triclinic=True), 5.0, 160, False, None),
    ("groups_of_eight_slots", dict(seed=24, n_systems=3, n_lo=1500, n_hi=2500, density=0.12), 6.0, 208, False, None),
    ("global_sort", dict(seed=25, n_systems=2, n_lo=5000, n_hi=9000, density=0.1), 5.0, 96, False, 2),
    ("per_system_sort", dict(seed=25, n_systems=2, n_lo=5000, n_hi=8000, density=0.1), 5.0, 96, False, 1),
    ("more_than_one_tile", dict(seed=26, n_systems=2, n_lo=2000, n_hi=3000, density=0.35), 6.0, 448, False, None),
]


@pytest.mark.parametrize("name,kw,rc,K,half,sort_path", CASES, ids=[c[0] for c in CASES])
def test_a_sequence_of_sparse_builds_leaves_what_fresh_builds_write(name, kw, rc, K, half, sort_path):
    pos, cell, pbc, ptr, bidx = system(**kw)
    N = pos.shape[0]
    kept = Buffers(N, K)
    g = torch.Generator().manual_seed(kw["seed"])
    skipped_some = False
    for step in range(6):
        build(pos, cell, pbc, ptr, bidx, rc, K, half, kept, sparse=True, sort_path=sort_path)
        want = fresh_build(pos, cell, pbc, ptr, bidx, rc, K, half, sort_path=sort_path)
        torch.cuda.synchronize()
        assert int(want.nn.max()) < K, "rows too short for this case"
        assert same_lists(kept, want, N), (name, step)
        # the record is true: where it says "zeros", there are zeros
        shift = 0
        while (K - 1) >> shift > 31:
            shift += 1
        slot_group = torch.arange(K, device=DEV) >> shift
        clean = ((kept.groups[:, None] >> slot_group[None, :]) & 1) == 0
        assert bool((kept.sh.abs().amax(2)[clean] == 0).all()), (name, step)
        skipped_some = skipped_some or bool(clean[kept.nm < N].any())
        drift(pos, cell, bidx, g, 0.6)
    if name == "more_than_one_tile":
        # (rows that the search finishes over several tiles are written whole and recorded as such)
        assert bool((kept.groups == -1).any())
    else:
        assert skipped_some, "the case never had a zero shift to leave out"


def test_selective_builds_keep_the_records_of_the_systems_they_skip():
    pos, cell, pbc, ptr, bidx = system(seed=27, n_systems=8, n_lo=300, n_hi=800, density=0.1)
    N, K, rc = pos.shape[0], 96, 5.0
    kept = Buffers(N, K)
    want = Buffers(N, K)
    g = torch.Generator().manual_seed(27)
    build(pos, cell, pbc, ptr, bidx, rc, K, False, kept, sparse=True)
    build(pos, cell, pbc, ptr, bidx, rc, K, False, want, sparse=False)
    for step in range(5):
        flags = (torch.rand(8, generator=g) < 0.5).to(DEV)
        drift(pos, cell, bidx, g, 0.6)
        build(pos, cell, pbc, ptr, bidx, rc, K, False, kept, sparse=True, flags=flags)
        build(pos, cell, pbc, ptr, bidx, rc, K, False, want, sparse=False, flags=flags)  # (tail_mode 1: whole tails)
        torch.cuda.synchronize()
        assert same_lists(kept, want, N), step


def test_after_a_foreign_write_every_word_set_makes_the_next_build_write_everything():
    pos, cell, pbc, ptr, bidx = system(seed=28, n_systems=4, n_lo=400, n_hi=900, density=0.1)
    N, K, rc = pos.shape[0], 96, 5.0
    kept = Buffers(N, K)
    build(pos, cell, pbc, ptr, bidx, rc, K, False, kept, sparse=True)
    kept.sh.fill_(7)  # (somebody else's write, over listed pairs and padding alike)
    kept.groups.fill_(-1)
    kept.nn.fill_(K)  # (and the padding of whole rows has to be restored, as tail_mode 0 does from the old counts)
    build(pos, cell, pbc, ptr, bidx, rc, K, False, kept, sparse=True)
    want = fresh_build(pos, cell, pbc, ptr, bidx, rc, K, False)
    torch.cuda.synchronize()
    assert same_lists(kept, want, N)


def test_the_hook_keeps_its_record_through_a_change_of_row_length():
    """NeighborListHook sizes its rows on the first call (and may trim them); every later call's shifts are those of
    a fresh build."""
    import sys
    sys.path.insert(0, ".")
    import bench
    from nvalchemi_amd.hooks._context import HookContext
    from nvalchemi_amd.models import LennardJonesModelWrapper

    g = torch.Generator().manual_seed(9)
    L = (5000 / 0.1) ** (1 / 3)  # (systems of more than 4096 atoms: the hook keeps the record for those only)
    batch = bench._batch_of([(torch.rand(5000, 3, generator=g) * L, torch.eye(3) * L) for _ in range(2)], torch.device(DEV))
    model = LennardJonesModelWrapper(epsilon=0.01, sigma=1.5, cutoff=6.0)
    hook = model.make_neighbor_hooks()[0]
    ctx = HookContext(batch=batch, model=model, workflow=None)
    for step in range(4):
        hook(ctx, hook.stage)
        K = hook._neighbor_matrix.shape[1]
        want = fresh_build(batch.positions, batch.cell, batch.pbc, batch.batch_ptr, batch.batch_idx, 6.0, K, False)
        torch.cuda.synchronize()
        got = Buffers.__new__(Buffers)
        got.nm, got.nn, got.sh = hook._neighbor_matrix, hook._num_neighbors, hook._neighbor_matrix_shifts
        assert same_lists(got, want, batch.num_nodes), step
        assert not hook._shift_groups_stale and (step == 0 or bool((hook._shift_groups != -1).any()))
        drift(batch.positions, batch.cell, batch.batch_idx, g, 0.5)


def test_what_the_entry_refuses():
    pos, cell, pbc, ptr, bidx = system(seed=29, n_systems=2, n_lo=100, n_hi=200, density=0.1)
    out = Buffers(pos.shape[0], 64)
    from nvalchemi_amd import _lib

    with pytest.raises(ValueError, match="tail_mode 0"):
        _lib.nl_build(pos, cell, pbc, ptr, bidx, None, 5.0, 64, False, 1, out.nm, out.nn, out.sh, shift_groups=out.groups)
    with pytest.raises(ValueError, match="float32"):
        _lib.nl_build(pos.double(), cell.double(), pbc, ptr, bidx, None, 5.0, 64, False, 0, out.nm, out.nn, out.sh,
                      shift_groups=out.groups)
