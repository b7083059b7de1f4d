"""GPU parity of the neighbor-list build (through the C ABI) against the CPU oracle.

Bar: bit-exact as canonically sorted (i, j, sx, sy, sz) sets; counts equal; every slot at or
beyond the count holds the padding (N / 0) -- the stale-slot rule of
nvalchemi/hooks/neighbor_list.py:377-380 and test/hooks/test_neighbor_list_hook.py:1031-1086.
"""

import numpy as np
import pytest
import torch

import oracle
from _systems import fcc_boxes, molecules_batch, periodic_batch, ptr_from_counts

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(autouse=True, params=["per_system", "global_sort"])
def sort_path(request, monkeypatch):
    """Every test runs twice: with the workgroup-per-system sort that batches of small systems
    take by default, and with the global histogram/scan/scatter pipeline that large systems take
    (nvamd_nl_build_path's sort_path argument, through the binding's default for it)."""
    from nvalchemi_amd import _lib

    monkeypatch.setattr(_lib, "nl_sort_path",
                        _lib.NL_SORT_GLOBAL if request.param == "global_sort" else _lib.NL_SORT_PER_SYSTEM)
    return request.param


def gpu_build(P, C, pb, ptr, rc, K, half=False, tail_mode=1, flags=None, prev=None):
    from nvalchemi_amd import _lib

    N = len(P)
    pos = torch.from_numpy(np.ascontiguousarray(P, dtype=np.float32)).to(DEV)
    cell = None if C is None else torch.from_numpy(np.ascontiguousarray(C, dtype=np.float32)).to(DEV)
    pbc = None if C is None else torch.from_numpy(np.ascontiguousarray(pb)).to(DEV)
    bptr = torch.from_numpy(np.asarray(ptr, dtype=np.int32)).to(DEV)
    bidx = torch.from_numpy(oracle.batch_idx_from_ptr(ptr)).to(DEV)
    if prev is None:
        nm = torch.full((N, K), N, dtype=torch.int32, device=DEV)
        nn = torch.zeros(N, dtype=torch.int32, device=DEV)
        sh = torch.zeros((N, K, 3), dtype=torch.int32, device=DEV) if C is not None else None
    else:
        nm, nn, sh = prev
    fl = None if flags is None else torch.tensor(flags, dtype=torch.bool, device=DEV)
    _lib.nl_build(pos, cell, pbc, bptr, bidx, fl, rc, K, half, tail_mode, nm, nn, sh)
    torch.cuda.synchronize()
    return nm, nn, sh


def check_against_oracle(P, C, pb, ptr, rc, half=False, K=None):
    ref = oracle.nl_brute(P, C, pb, ptr, rc, half=half)
    N = len(P)
    counts = np.bincount(ref[:, 0], minlength=N) if len(ref) else np.zeros(N, dtype=np.int64)
    if K is None:
        K = int(counts.max()) + 1 if N else 1
    nm, nn, sh = gpu_build(P, C, pb, ptr, rc, K, half=half)
    nm_, nn_ = nm.cpu().numpy(), nn.cpu().numpy()
    sh_ = None if sh is None else sh.cpu().numpy()
    assert np.array_equal(nn_, counts)
    got = oracle.matrix_to_edges(nm_, nn_, sh_)
    assert np.array_equal(got, ref)
    cols = np.arange(K)[None, :]
    tail = cols >= nn_[:, None]
    assert np.all(nm_[tail] == N)
    if sh_ is not None:
        assert np.all(sh_[tail] == 0)
    return nm, nn, sh


def test_line_and_periodic_image_known_answers():
    line = np.array([[0.0, 0, 0], [1.5, 0, 0], [5.0, 0, 0]], dtype=np.float32)
    nm, nn, _ = gpu_build(np.concatenate([line, line]), None, None, [0, 3, 6], 2.5, 4)
    assert nn.tolist() == [1, 1, 0, 1, 1, 0]
    assert nm[:, 0].tolist() == [1, 0, 6, 4, 3, 6]
    pos = np.array([[0.1, 0, 0], [2.9, 0, 0]], dtype=np.float32)
    cell = np.eye(3, dtype=np.float32)[None] * 3.0
    nm, nn, sh = gpu_build(pos, cell, np.ones((1, 3), bool), [0, 2], 2.5, 4)
    assert nn.tolist() == [1, 1] and nm[:, 0].tolist() == [1, 0]
    assert sh[0, 0].tolist() == [-1, 0, 0] and sh[1, 0].tolist() == [1, 0, 0]


CASES = [
    dict(seed=1, n_systems=5, n_lo=20, n_hi=300, density=0.05, triclinic=False, rc=5.0),
    dict(seed=2, n_systems=6, n_lo=8, n_hi=200, density=0.0764, triclinic=True, rc=5.0),
    dict(seed=3, n_systems=4, n_lo=8, n_hi=40, density=0.0764, triclinic=True, rc=6.0, spread=2.0),
    dict(seed=4, n_systems=3, n_lo=50, n_hi=400, density=0.1, triclinic=False, rc=6.0,
         pbc=[True, True, False]),
    dict(seed=5, n_systems=3, n_lo=1, n_hi=3, density=0.2, triclinic=True, rc=4.0),
    dict(seed=6, n_systems=16, n_lo=8, n_hi=2000, density=0.0764, triclinic=True, rc=5.0),
    dict(seed=7, n_systems=2, n_lo=3000, n_hi=4000, density=0.8, triclinic=False, rc=2.5),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"seed{c['seed']}")
@pytest.mark.parametrize("half", [False, True])
def test_random_periodic_batches_match_brute_force(case, half):
    c = dict(case)
    rc = c.pop("rc")
    if half and c["seed"] in (6, 7):
        pytest.skip("half lists are covered by the smaller cases")
    P, C, pb, ptr = periodic_batch(**c)
    check_against_oracle(P, C, pb, ptr, rc, half=half)


def test_a_batch_whose_mean_system_takes_the_sort_with_eight_atoms_per_lane():
    """Systems of 300 to 6000 atoms with a mean between 2049 and 4096: the per-system sort keeps eight atoms per lane
    in registers for those that fit (up to 4096 atoms) and bins the larger one twice; triclinic cells."""
    from _systems import ptr_from_counts, random_triclinic_cell

    rng = np.random.default_rng(31)
    counts = [300, 3900, 4700, 2200, 4096]
    cells, pos = [], []
    for n in counts:
        H = random_triclinic_cell(rng, (n / 0.8) ** (1.0 / 3.0))
        pos.append((rng.uniform(0, 1, (n, 3)) @ H.astype(np.float64)).astype(np.float32))
        cells.append(H)
    P, C = np.concatenate(pos), np.stack(cells).astype(np.float32)
    check_against_oracle(P, C, np.ones((len(counts), 3), dtype=bool), ptr_from_counts(counts), 2.5)


def test_molecules_without_cell():
    P, Z, M, ptr = molecules_batch(seed=0)
    check_against_oracle(P, None, None, ptr, 5.0, K=32)


def test_non_periodic_flags_with_a_cell_do_not_wrap():
    P, C, pb, ptr = periodic_batch(12, 3, 30, 60, 0.05, spread=0.4)
    pb[:] = False
    check_against_oracle(P, C, pb, ptr, 5.0)


def test_fcc_boxes_rc6():
    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=3, reps=5)
    nm, nn, sh = check_against_oracle(P, C, pb, ptr, 6.0)
    assert int(nn.min()) >= 70 and int(nn.max()) <= 86


def test_tiny_cell_many_images_and_self_images():
    rng = np.random.default_rng(0)
    P = rng.uniform(0, 2.0, (3, 3)).astype(np.float32)
    C = (np.eye(3, dtype=np.float32) * np.array([2.0, 2.3, 1.9], dtype=np.float32))[None]
    check_against_oracle(P, C, np.ones((1, 3), bool), [0, 3], 4.5)


def test_atoms_many_cells_away_take_the_unpacked_shift_path():
    """Shifts travel through the search as three 5-bit fields; an atom that sits 20 to 40 cell lengths
    outside its cell has a wider one, which is recovered from the sorted arrays instead.  (Multiples of
    lattice vectors that float32 adds exactly: edge lengths are powers of two.)"""
    rng = np.random.default_rng(5)
    counts = [40, 70]
    C = np.stack([np.diag([8.0, 8.0, 16.0]), np.array([[8.0, 0, 0], [2.0, 8.0, 0], [0, 4.0, 16.0]])]).astype(np.float32)
    pos = []
    for n, H in zip(counts, C):
        f = rng.uniform(0, 1, (n, 3))
        hop = rng.integers(-40, 41, (n, 3)) * (rng.random((n, 1)) < 0.5)
        pos.append(((f + hop) @ H.astype(np.float64)).astype(np.float32))
    P = np.concatenate(pos)
    pb = np.ones((2, 3), bool)
    nm, nn, sh = check_against_oracle(P, C, pb, ptr_from_counts(counts), 5.0)
    assert int(sh.abs().max()) > 15
    check_against_oracle(P, C, pb, ptr_from_counts(counts), 5.0, half=True)


@pytest.mark.parametrize("seed", range(24))
def test_pairs_within_a_hair_of_the_cutoff(seed):
    """Pairs placed at rc (1 +- 10^-7.5 .. 10^-4) in cells from a fraction of the cutoff to six cutoffs wide,
    skewed or not, atoms up to two cells outside: every one of them lies inside one of the float32 uncertainty
    bands of the search (the scan's expanded form has the wider one) and has to come out as the double-precision
    expression on the float32 inputs decides."""
    rng = np.random.default_rng(7000 + seed)
    rc = float(rng.choice([1.0, 2.5, 5.0]))
    L = rc * rng.uniform(0.6, 6.0, 3)
    H = np.diag(L)
    if rng.random() < 0.7:
        H[1, 0] = rng.uniform(-0.5, 0.5) * L[0]
        H[2, 0] = rng.uniform(-0.5, 0.5) * L[0]
        H[2, 1] = rng.uniform(-0.5, 0.5) * L[1]
    n_pairs = int(rng.integers(20, 120))
    base = rng.uniform(-1.0, 2.0, (n_pairs, 3)) @ H
    dirs = rng.normal(size=(n_pairs, 3))
    dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
    eps = 10.0 ** rng.uniform(-7.5, -4.0, n_pairs) * rng.choice([-1.0, 1.0], n_pairs)
    P = np.concatenate([base, base + dirs * (rc * (1.0 + eps))[:, None]]).astype(np.float32)
    pb = (rng.random(3) < 0.8)[None]
    check_against_oracle(P, H.astype(np.float32)[None], pb, ptr_from_counts([len(P)]), rc)


def test_empty_systems_and_single_atoms():
    pos = np.array([[0.0, 0, 0], [1.0, 0, 0], [9.0, 9, 9]], dtype=np.float32)
    check_against_oracle(pos, None, None, ptr_from_counts([0, 2, 0, 1]), 2.0, K=4)


def test_overflow_counts_past_k_without_writing_past_k():
    P, C, pb, ptr = periodic_batch(21, 2, 80, 120, 0.1)
    ref = oracle.nl_brute(P, C, pb, ptr, 5.0)
    counts = np.bincount(ref[:, 0], minlength=len(P))
    K = 8
    assert counts.max() > K
    N = len(P)
    guard = torch.full((N + 1, K), -7, dtype=torch.int32, device=DEV)
    nm = guard[:N]
    nm.fill_(N)
    nn = torch.zeros(N, dtype=torch.int32, device=DEV)
    sh = torch.zeros((N, K, 3), dtype=torch.int32, device=DEV)
    gpu_build(P, C, pb, ptr, 5.0, K, prev=(nm, nn, sh))
    assert np.array_equal(nn.cpu().numpy(), counts)
    assert torch.all(guard[N] == -7)
    # every written entry is a true neighbor
    got = oracle.matrix_to_edges(nm.cpu().numpy(), nn.cpu().numpy(), sh.cpu().numpy())
    refset = {tuple(r) for r in ref.tolist()}
    assert all(tuple(r) in refset for r in got.tolist())


def test_persistent_buffers_keep_padding_and_selective_rebuild():
    P, C, pb, ptr = periodic_batch(31, 3, 40, 60, 0.08)
    rc = 5.0
    ref = oracle.nl_brute(P, C, pb, ptr, rc)
    K = int(np.bincount(ref[:, 0], minlength=len(P)).max()) + 3
    bufs = gpu_build(P, C, pb, ptr, rc, K, tail_mode=0)
    # move system 1 apart (dilate): fewer neighbors; rebuild only system 1
    P2 = P.copy()
    a0, a1 = ptr[1], ptr[2]
    C2 = C.copy()
    P2[a0:a1] *= 1.5
    C2[1] *= 1.5
    before = [t.clone() for t in bufs]
    gpu_build(P2, C2, pb, ptr, rc, K, tail_mode=0, flags=[False, True, False], prev=bufs)
    nm, nn, sh = (t.cpu().numpy() for t in bufs)
    ref2 = oracle.nl_brute(P2, C2, pb, ptr, rc)
    sel = (ref2[:, 0] >= a0) & (ref2[:, 0] < a1)
    keep = (ref[:, 0] < a0) | (ref[:, 0] >= a1)
    expect = oracle.canonical_edges(np.concatenate([ref[keep], ref2[sel]]))
    assert np.array_equal(oracle.matrix_to_edges(nm, nn, sh), expect)
    cols = np.arange(K)[None, :]
    tail = cols >= nn[:, None]
    assert np.all(nm[tail] == len(P)) and np.all(sh[tail] == 0)
    # untouched systems are bit-identical, slot by slot
    for t_new, t_old in zip(bufs, before):
        assert torch.equal(t_new[:a0], t_old[:a0]) and torch.equal(t_new[a1:], t_old[a1:])


def test_repeated_builds_are_identical_as_sets():
    P, C, pb, ptr = periodic_batch(41, 4, 200, 400, 0.5)
    a = gpu_build(P, C, pb, ptr, 2.5, 64)
    b = gpu_build(P, C, pb, ptr, 2.5, 64)
    ea = oracle.matrix_to_edges(*(t.cpu().numpy() for t in a))
    eb = oracle.matrix_to_edges(*(t.cpu().numpy() for t in b))
    assert np.array_equal(ea, eb)


def test_per_system_path_with_a_system_too_large_for_its_lds_histogram(sort_path):
    """A batch whose mean system size selects the workgroup-per-system sort, with one system whose
    cell count exceeds the LDS histogram (8192 cells): that system goes through global memory."""
    rng = np.random.default_rng(11)
    counts = [5, 20000, 0, 7, 300]
    L_big = 60.0  # cutoff 2.0: 29^3 cells, halved once along x to fit the cap of 20000: 12615 > 8192
    P, C, pb = [], [], []
    for n in counts:
        L = L_big if n > 1000 else 6.0
        P.append(rng.uniform(0, L, size=(n, 3)))
        C.append(np.eye(3) * L)
        pb.append([True, True, True])
    P = np.concatenate(P).astype(np.float32)
    C = np.stack(C).astype(np.float32)
    pb = np.array(pb, dtype=bool)
    ptr = ptr_from_counts(counts)
    rc = 2.0
    K = 96  # the 300 atoms in the 6^3 box are the dense ones (about 46 neighbors on average)
    nm_r, nn_r, sh_r = oracle.nl_cell(P, C, pb, ptr, rc, K)
    assert nn_r.max() < K
    ref = oracle.matrix_to_edges(nm_r, nn_r, sh_r)
    nm, nn, sh = gpu_build(P, C, pb, ptr, rc, K)
    assert np.array_equal(nn.cpu().numpy(), nn_r)
    got = oracle.matrix_to_edges(nm.cpu().numpy(), nn.cpu().numpy(), sh.cpu().numpy())
    assert np.array_equal(got, ref)
