"""Seeded random sweep of the neighbor build and the pair kernel against the oracle: cell shapes
from cubic to strongly sheared, cutoffs from a fraction of the cell to several cells (many
images), every pattern of periodic axes, empty and one-atom systems, coordinates far outside the
cell, full and half lists, selective rebuilds over stale buffers.  Each case is small (the
brute-force oracle is the checker); the seeds are fixed, so a failure names its case."""

import numpy as np
import pytest
import torch

import oracle
from _systems import ptr_from_counts

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def random_case(seed):
    rng = np.random.default_rng(1000 + seed)
    n_sys = int(rng.integers(1, 7))
    counts = rng.choice([0, 1, 2, 3, 5, 9, 17, 40, 90], n_sys)
    if counts.sum() == 0:
        counts[0] = 4
    periodic = rng.random() < 0.8
    cells, pos, pbcs = [], [], []
    for n in counts:
        L = rng.uniform(2.0, 9.0, 3)
        H = np.diag(L)
        if rng.random() < 0.6:  # shear, up to strongly skewed but well conditioned
            H[1, 0] = rng.uniform(-0.6, 0.6) * L[0]
            H[2, 0] = rng.uniform(-0.5, 0.5) * L[0]
            H[2, 1] = rng.uniform(-0.5, 0.5) * L[1]
        if rng.random() < 0.3:  # any right-handed or left-handed row order
            H = H[rng.permutation(3)]
        spread = rng.choice([0.0, 0.0, 0.7, 3.0])
        f = rng.uniform(-spread, 1.0 + spread, (n, 3))
        pos.append((f @ H).astype(np.float32))
        cells.append(H.astype(np.float32))
        pbcs.append(rng.random(3) < 0.75)
    P = np.concatenate(pos).astype(np.float32).reshape(-1, 3)
    C = np.stack(cells)
    pb = np.stack(pbcs)
    rc = float(rng.choice([0.9, 1.7, 2.6, 4.1, 6.5]))
    half = bool(rng.random() < 0.3)
    if not periodic:
        C, pb = None, None
    return P, C, pb, ptr_from_counts(counts), rc, half


def T(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a), device=DEV)
    return t if dtype is None else t.to(dtype)


@pytest.mark.parametrize("seed", range(200))
def test_random_case(seed, monkeypatch):
    from nvalchemi_amd import _lib

    monkeypatch.setattr(_lib, "nl_sort_path", _lib.NL_SORT_GLOBAL if seed % 2 else _lib.NL_SORT_PER_SYSTEM)
    P, C, pb, ptr, rc, half = random_case(seed)
    N, B = len(P), len(ptr) - 1
    ref = oracle.nl_brute(P, C, pb, ptr, rc, half=half)
    counts = np.bincount(ref[:, 0], minlength=N) if len(ref) else np.zeros(N, dtype=np.int64)
    if counts.max(initial=0) > 1500:
        pytest.skip("more images than a small case should have")
    K = int(counts.max(initial=0)) + 1 + seed % 3
    bidx = oracle.batch_idx_from_ptr(ptr)
    # stale buffers: another build's leftovers that the new one must overwrite or clear
    nm = torch.full((N, K), 7 % max(N, 1), dtype=torch.int32, device=DEV)
    nn = torch.full((N,), K, dtype=torch.int32, device=DEV)
    sh = torch.full((N, K, 3), 3, dtype=torch.int32, device=DEV) if C is not None else None
    args = (T(P), None if C is None else T(C), None if C is None else T(pb), T(ptr), T(bidx))
    _lib.nl_build(*args, None, rc, K, half, 1, nm, nn, sh)
    nm_, nn_ = nm.cpu().numpy(), nn.cpu().numpy()
    sh_ = None if sh is None else sh.cpu().numpy()
    assert np.array_equal(nn_, counts), (seed, rc, half)
    assert np.array_equal(oracle.matrix_to_edges(nm_, nn_, sh_), ref), (seed, rc, half)
    tail = np.arange(K)[None, :] >= nn_[:, None]
    assert np.all(nm_[tail] == N) and (sh_ is None or np.all(sh_[tail] == 0))

    # a selective rebuild after moving every atom: flagged systems follow, the others keep their rows
    if B > 1:
        rng = np.random.default_rng(seed)
        flags = rng.random(B) < 0.5
        P2 = (P + rng.normal(0, 0.3, P.shape)).astype(np.float32)
        before = (nm.clone(), nn.clone(), None if sh is None else sh.clone())
        _lib.nl_build(T(P2), *args[1:], T(flags), rc, K + 0, half, 0, nm, nn, sh)
        ref2 = oracle.nl_brute(P2, C, pb, ptr, rc, half=half)
        cnt2 = np.bincount(ref2[:, 0], minlength=N) if len(ref2) else np.zeros(N, dtype=np.int64)
        rows = flags[bidx]
        got_n = nn.cpu().numpy()
        assert np.array_equal(got_n[rows], cnt2[rows]) and np.array_equal(got_n[~rows], counts[~rows])
        if cnt2.max(initial=0) < K:
            got = oracle.matrix_to_edges(nm.cpu().numpy(), got_n, None if sh is None else sh.cpu().numpy())
            keep_new = rows[ref2[:, 0]] if len(ref2) else np.zeros(0, bool)
            keep_old = ~rows[ref[:, 0]] if len(ref) else np.zeros(0, bool)
            want = np.concatenate([ref2[keep_new], ref[keep_old]])
            want = want[np.lexsort(want.T[::-1])]
            assert np.array_equal(got, want), (seed, "selective")
        assert torch.equal(nm[T(~rows)], before[0][T(~rows)])

    # the pair kernel on that list (full lists: with and without derived shifts)
    if N and len(ref):
        _lib.nl_build(*args, None, rc, K, half, 1, nm, nn, sh)
        cells = C if C is not None else np.eye(3, dtype=np.float32)[None].repeat(B, 0)
        want = oracle.lj_matrix(P, cells, nm_, sh_, nn_, bidx, N, 0.3, 0.8 * rc / 2.5, rc, half=half, virial=True)
        for hint in ((0.0,) if half else (0.0, rc)):
            e, f = torch.empty(N, device=DEV), torch.empty((N, 3), device=DEV)
            w, es = torch.empty((B, 9), device=DEV), torch.empty(B, device=DEV)
            _lib.lj_energy_forces(T(P), T(cells), nm, sh, nn, T(bidx), N, 0.3, 0.8 * rc / 2.5, rc, 0.0, half, e, f, w, es,
                                  neighbor_list_cutoff=hint)
            fr = want["forces"].astype(np.float64)
            scale = max(1.0, float(np.abs(fr).max()))
            assert np.abs(f.cpu().numpy() - fr).max() <= 1e-6 + 1e-5 * scale, (seed, hint)
            er = want["energy"].astype(np.float64)
            assert np.abs(es.cpu().numpy() - er).max() <= 1e-6 + 1e-5 * max(1.0, float(np.abs(er).max())), (seed, hint)
