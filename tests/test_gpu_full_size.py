"""GPU checks at the sizes the headline configurations are quoted on.

Where the CPU oracle finishes in seconds (the 32 000-atom FCC batch; samples of the larger ones)
results are compared with it directly, to the usual bars (neighbor data bit-exact as sorted sets,
float32 energies and forces to 1e-5 relative / 1e-6 absolute).  Beyond that, size-independent
properties are checked on the whole output: the full list is symmetric ((i, j, S) present iff
(j, i, -S) is), rows of sampled atoms equal a brute-force search over all atoms, forces of every
system sum to zero, per-system energies and the virial trace equal an independent float64 torch
evaluation over the edge list, and the flat indexing works past 2^31 elements.
"""

import math

import numpy as np
import pytest
import torch

import oracle
from _systems import fcc_boxes, periodic_batch, ptr_from_counts, random_triclinic_cell

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def build_on_gpu(pos, cell, pbc, ptr, rc, K):
    from nvalchemi_amd import _lib

    N, B = pos.shape[0], ptr.shape[0] - 1
    bidx = torch.repeat_interleave(torch.arange(B, dtype=torch.int32, device=DEV),
                                   (ptr[1:] - ptr[:-1]).long())
    nm = torch.full((N, K), N, dtype=torch.int32, device=DEV)
    nn = torch.zeros(N, dtype=torch.int32, device=DEV)
    sh = torch.zeros((N, K, 3), dtype=torch.int32, device=DEV)
    _lib.nl_build(pos, cell, pbc, ptr, bidx, None, rc, K, False, 1, nm, nn, sh)
    torch.cuda.synchronize()
    return nm, nn, sh, bidx


def edge_list(nm, nn, sh):
    """(i, j, S) of every used slot, as torch tensors on the device."""
    N, K = nm.shape
    used = torch.arange(K, device=DEV)[None, :] < nn.clamp(max=K)[:, None]
    i = torch.arange(N, device=DEV)[:, None].expand(N, K)[used]
    return i, nm[used].long(), sh[used].long()


def assert_symmetric(i, j, S, N):
    assert int(S.abs().max()) <= 1
    code = (S[:, 0] + 1) * 9 + (S[:, 1] + 1) * 3 + (S[:, 2] + 1)
    back = (1 - S[:, 0]) * 9 + (1 - S[:, 1]) * 3 + (1 - S[:, 2])
    fwd = ((i * N + j) * 27 + code).sort().values
    rev = ((j * N + i) * 27 + back).sort().values
    assert torch.equal(fwd, rev)
    assert not bool((fwd[1:] == fwd[:-1]).any()), "an edge is listed twice"


def rows_equal_brute_force(pos, cell_row, rc, nm, nn, sh, atoms, lo, hi):
    """Rows of the given atoms against a float64 search over all atoms lo..hi of their (cubic,
    fully periodic, L > 2 rc) system, with the pair separation in the kernel's association."""
    L = float(cell_row[0, 0])
    p = pos[lo:hi].double()
    for a in atoms:
        d = p - pos[a].double()
        S = -torch.round(d / L)
        d = d + S * L
        r2 = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
        hit = (r2 < rc * rc)
        hit[a - lo] = False
        assert float((r2[hit].max() if hit.any() else 0.0)) < rc * rc
        # no candidate may sit so close to the cutoff that the two evaluations could disagree
        assert float((r2 - rc * rc).abs().min()) > 1e-9, "sample again: a pair lies on the cutoff"
        want = {(int(j) + lo, int(s[0]), int(s[1]), int(s[2])) for j, s in zip(hit.nonzero().ravel().tolist(), S[hit].long().tolist())}
        n = int(nn[a])
        got = {(int(j), *map(int, s)) for j, s in zip(nm[a, :n].tolist(), sh[a, :n].tolist())}
        assert got == want, a


def torch_lj_over_edges(pos, cell, bidx, i, j, S, eps, sig, rc, B):
    """float64 LJ energies per system, forces per atom and virial trace per system from an edge list,
    and per atom the sum of the magnitudes of its pair-force terms (what bounds the rounding error of
    any float64 accumulation of them, in whatever order)."""
    h = cell.double()[bidx[i].long()]
    d = (pos[j].double() - pos[i].double()) + torch.einsum("ek,ekc->ec", S.double(), h)
    r2 = (d * d).sum(1)
    inside = r2 < rc * rc
    q6 = (sig * sig / r2) ** 3
    u = torch.where(inside, 4 * eps * (q6 * q6 - q6), torch.zeros_like(r2))
    g = torch.where(inside, -24 * eps * (2 * q6 * q6 - q6) / r2, torch.zeros_like(r2))  # u'(r)/r
    e_sys = torch.zeros(B, dtype=torch.float64, device=DEV).index_add_(0, bidx[i].long(), 0.5 * u)
    f = torch.zeros(pos.shape[0], 3, dtype=torch.float64, device=DEV).index_add_(0, i, g[:, None] * d)
    f_terms = torch.zeros(pos.shape[0], dtype=torch.float64, device=DEV).index_add_(0, i, (g[:, None] * d).abs().sum(1))
    w_tr = torch.zeros(B, dtype=torch.float64, device=DEV).index_add_(0, bidx[i].long(), -0.5 * g * r2)
    return e_sys, f, w_tr, f_terms


def close(got, want, slack=None):
    """|got - want| <= 1e-6 + 1e-5 |want| (the bar for float32 energies and forces), elementwise;
    ``slack`` adds an absolute allowance per element where the test says why."""
    tol = 1e-6 + 1e-5 * want.abs()
    if slack is not None:
        tol = tol + slack
    return bool(((got.double() - want).abs() <= tol).all())


def gpu_lj(pos, cell, nm, sh, nn, bidx, eps, sig, rc, virial, neighbor_list_cutoff=0.0):
    """``neighbor_list_cutoff`` > 0 is the hinted call: in cells wide enough the kernel derives the
    shifts from the positions instead of reading them."""
    from nvalchemi_amd import _lib

    N, B = pos.shape[0], cell.shape[0]
    e = torch.empty(N, dtype=torch.float32, device=DEV)
    f = torch.empty((N, 3), dtype=torch.float32, device=DEV)
    w = torch.empty((B, 9), dtype=torch.float32, device=DEV) if virial else None
    es = torch.empty(B, dtype=torch.float32, device=DEV)
    _lib.lj_energy_forces(pos, cell, nm, sh, nn, bidx, N, eps, sig, rc, 0.0, False, e, f, w, es,
                          neighbor_list_cutoff=neighbor_list_cutoff)
    torch.cuda.synchronize()
    return e, f, w, es


def test_fcc_batch_of_64_boxes_against_the_oracle():
    """64 periodic FCC boxes of 500 atoms, cutoff 6: small enough for the oracle as a whole."""
    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=64, reps=5, a=3.6, jitter=0.05)
    rc, K = 6.0, 96
    sig = (3.6 / math.sqrt(2)) / 2 ** (1 / 6)
    nm_r, nn_r, sh_r = oracle.nl_cell(P, C, pb, ptr, rc, K)
    assert nn_r.max() < K and abs(nn_r.mean() - 78) < 1.0  # the five FCC shells inside 6
    pos, cell = torch.from_numpy(P).to(DEV), torch.from_numpy(C).to(DEV)
    nm, nn, sh, bidx = build_on_gpu(pos, cell, torch.from_numpy(pb).to(DEV), torch.from_numpy(ptr).to(DEV), rc, K)
    assert np.array_equal(nn.cpu().numpy(), nn_r)
    assert np.array_equal(oracle.matrix_to_edges(nm.cpu().numpy(), nn.cpu().numpy(), sh.cpu().numpy()),
                          oracle.matrix_to_edges(nm_r, nn_r, sh_r))
    ref = oracle.lj_matrix(P, C, nm_r, sh_r, nn_r, oracle.batch_idx_from_ptr(ptr), len(P), 0.01, sig, rc)
    e, f, _, es = gpu_lj(pos, cell, nm, sh, nn, bidx, 0.01, sig, rc, virial=False)
    for got, want in ((e, ref["atomic_energies"]), (f, ref["forces"]), (es, ref["energy"])):
        g, w = got.cpu().numpy().astype(np.float64), want.astype(np.float64)
        assert (np.abs(g - w) <= 1e-6 + 1e-5 * np.abs(w)).all()


def relaxed_liquid(B, n, rho, rc, steps=50):
    """The quoted workload's own preparation: uniform random positions (seed 0) relaxed by 50 FIRE steps
    (dt 0.005, maxstep 0.07 sigma, as bench.py does) of the package's own FIRE over its own neighbor hook and model."""
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.dynamics import FIRE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    L = (n / rho) ** (1 / 3)
    g = torch.Generator().manual_seed(0)
    data = [AtomicData(torch.rand(n, 3, generator=g) * L, torch.full((n,), 18, dtype=torch.long),
                       atomic_masses=torch.ones(n), cell=torch.eye(3) * L, pbc=torch.tensor([True, True, True]),
                       forces=torch.zeros(n, 3), energy=torch.zeros(1, 1)) for _ in range(B)]
    batch = Batch.from_data_list(data, device=DEV)
    model = LennardJonesModelWrapper(epsilon=1.0, sigma=1.0, cutoff=rc)
    FIRE(model, dt=0.005, maxstep=0.07, hooks=model.make_neighbor_hooks()).run(batch, n_steps=steps)
    torch.cuda.synchronize()
    return batch.positions.detach().clone().contiguous(), batch.cell.detach().clone().contiguous(), L


def test_one_million_atom_liquid_batch():
    """256 boxes x 3900 atoms, density 0.8, cutoff 2.5, uniform random positions relaxed by 50 FIRE steps
    (the configuration the metric is quoted on), with the pair kernel called the way the timed step
    calls it: ``neighbor_list_cutoff = rc``, i.e. shifts derived from the positions in these cells."""
    B, n, rho, rc, K = 256, 3900, 0.8, 2.5, 112
    eps, sig = 1.0, 1.0
    pos, cell, L = relaxed_liquid(B, n, rho, rc)
    assert bool(torch.isfinite(pos).all())
    pbc = torch.ones(B, 3, dtype=torch.bool, device=DEV)
    ptr = (torch.arange(B + 1, dtype=torch.int32) * n).to(DEV)
    N = B * n
    nm, nn, sh, bidx = build_on_gpu(pos, cell, pbc, ptr, rc, K)
    assert int(nn.max()) < K
    assert abs(float(nn.float().mean()) - 4 / 3 * math.pi * rc ** 3 * rho) < 1.5  # (a liquid is not an ideal gas: the excluded core takes a little from the count)
    i, j, S = edge_list(nm, nn, sh)
    assert bool((bidx[i] == bidx[j]).all())
    assert_symmetric(i, j, S, N)
    e, f, w, es = gpu_lj(pos, cell, nm, sh, nn, bidx, eps, sig, rc, virial=True, neighbor_list_cutoff=rc)
    assert bool(torch.isfinite(es).all()) and bool(torch.isfinite(f).all()) and bool(torch.isfinite(w).all())
    # three whole boxes against the oracle: list bit-exact, energies / forces / virial to 1e-5 / 1e-6
    for s in (0, 101, 255):
        lo, hi = s * n, (s + 1) * n
        P1 = pos[lo:hi].cpu().numpy()
        C1 = cell[s:s + 1].cpu().numpy()
        nm_r, nn_r, sh_r = oracle.nl_cell(P1, C1, np.ones((1, 3), bool), np.array([0, n], np.int32), rc, K)
        got_nm = nm[lo:hi].cpu().numpy().copy()
        got_nm[got_nm < N] -= lo
        got_nm[got_nm == N] = n
        assert np.array_equal(nn[lo:hi].cpu().numpy(), nn_r)
        assert np.array_equal(oracle.matrix_to_edges(got_nm, nn_r, sh[lo:hi].cpu().numpy()),
                              oracle.matrix_to_edges(nm_r, nn_r, sh_r))
        ref = oracle.lj_matrix(P1, C1, nm_r, sh_r, nn_r, np.zeros(n, np.int32), n, eps, sig, rc, virial=True)
        for got, want in ((e[lo:hi], ref["atomic_energies"]), (f[lo:hi], ref["forces"]), (es[s:s + 1], ref["energy"]),
                          (w[s:s + 1], ref["virials"])):
            assert close(got.cpu(), torch.from_numpy(want.astype(np.float64)).reshape(got.shape)), s
    # the hinted call against the call that reads the shifts: per-atom results bit for bit
    e0, f0, w0, es0 = gpu_lj(pos, cell, nm, sh, nn, bidx, eps, sig, rc, virial=True)
    assert torch.equal(e0, e) and torch.equal(f0, f)
    assert close(es0, es.double()) and close(w0, w.double())
    # every system against a float64 torch evaluation over the edge list.  Forces: the bar, plus the
    # rounding of a float64 sum of the atom's pair terms (1e-13 of the sum of their magnitudes; it only
    # matters for an atom whose large terms cancel)
    e_sys, f64, w_tr, f_terms = torch_lj_over_edges(pos, cell, bidx, i, j, S, eps, sig, rc, B)
    assert close(es, e_sys)
    assert close(f, f64, slack=1e-13 * f_terms[:, None])
    assert close(w.double()[:, 0] + w.double()[:, 4] + w.double()[:, 8], w_tr)
    # Newton's third law per system, relative to the size of the terms that cancel
    fsum = torch.zeros(B, 3, dtype=torch.float64, device=DEV).index_add_(0, bidx.long(), f.double())
    fabs = torch.zeros(B, dtype=torch.float64, device=DEV).index_add_(0, bidx.long(), f.double().abs().sum(1))
    assert bool((fsum.abs().max(1).values <= 1e-6 * fabs + 1e-3).all())


def test_inflight_mix_of_2048_triclinic_systems():
    """2048 triclinic cells of 8-2000 atoms (log-uniform), cutoff 5: the per-system sort with very
    different system sizes; neighbor counts of every atom and the full lists of sampled systems
    against the oracle; a masked FIRE step leaves inactive systems bit-identical."""
    rng = np.random.default_rng(0)
    Bn = 2048
    counts = np.exp(rng.uniform(np.log(8), np.log(2000), Bn)).astype(np.int64)
    cells, pos = [], []
    for n in counts:
        Lc = (n / 0.0764) ** (1 / 3)
        H = random_triclinic_cell(rng, Lc)
        cells.append(H)
        pos.append((rng.uniform(0, 1, (n, 3)) @ H.astype(np.float64)).astype(np.float32))
    P, C = np.concatenate(pos), np.stack(cells).astype(np.float32)
    pb = np.ones((Bn, 3), bool)
    ptr = ptr_from_counts(counts)
    rc, K = 5.0, 256  # the smallest cells are narrower than the cutoff: many images per atom
    oracle.set_threads(16)
    nm_r, nn_r, sh_r = oracle.nl_cell(P, C, pb, ptr, rc, K)
    assert nn_r.max() < K
    posd, celld = torch.from_numpy(P).to(DEV), torch.from_numpy(C).to(DEV)
    nm, nn, sh, bidx = build_on_gpu(posd, celld, torch.from_numpy(pb).to(DEV), torch.from_numpy(ptr).to(DEV), rc, K)
    assert np.array_equal(nn.cpu().numpy(), nn_r)
    nm_c, sh_c = nm.cpu().numpy(), sh.cpu().numpy()
    for s in rng.choice(Bn, 120, replace=False):
        lo, hi = ptr[s], ptr[s + 1]
        assert np.array_equal(oracle.matrix_to_edges(nm_c[lo:hi], nn_r[lo:hi], sh_c[lo:hi]),
                              oracle.matrix_to_edges(nm_r[lo:hi], nn_r[lo:hi], sh_r[lo:hi])), s
    # masked FIRE step at this size
    from nvalchemi_amd import _lib

    N = len(P)
    M = Bn
    f32 = lambda v: torch.full((M,), v, dtype=torch.float32, device=DEV)  # noqa: E731
    vel = torch.randn(N, 3, device=DEV) * 0.01
    forces = torch.randn(N, 3, device=DEV)
    masses = torch.ones(N, device=DEV)
    active = torch.from_numpy(rng.random(M) < 0.5).to(DEV)
    p0, v0 = posd.clone(), vel.clone()
    alpha, dt = f32(0.1), f32(0.01)
    npos = torch.zeros(M, dtype=torch.int32, device=DEV)
    a0, d0, n0 = alpha.clone(), dt.clone(), npos.clone()
    vf, vv, ff = f32(0), f32(0), f32(0)
    _lib.fire_step(posd, vel, forces, masses, alpha, dt, f32(0.1), f32(0.99), f32(0.001), f32(0.1), f32(0.2),
                   npos, torch.full((M,), 5, dtype=torch.int32, device=DEV), f32(0.5), f32(1.1),
                   torch.zeros(M, dtype=torch.int32, device=DEV), vf, vv, ff, bidx, True, active)
    torch.cuda.synchronize()
    frozen = ~active[bidx.long()]
    assert torch.equal(posd[frozen], p0[frozen]) and torch.equal(vel[frozen], v0[frozen])
    assert torch.equal(alpha[~active], a0[~active]) and torch.equal(dt[~active], d0[~active])
    assert torch.equal(npos[~active], n0[~active])
    moved = (posd[~frozen] != p0[~frozen]).any(1)
    assert float(moved.float().mean()) > 0.99


def test_four_million_atom_single_box():
    """One periodic box of 4 M atoms, density 0.1, cutoff 6: the global sort path, flat indices
    past 2^31 elements (K = 192), float64 per-system energy and virial."""
    N, rho, rc, K = 4_000_000, 0.1, 6.0, 192
    L = (N / rho) ** (1 / 3)
    g = torch.Generator().manual_seed(0)
    pos = (torch.rand(N, 3, generator=g) * L).to(DEV)
    cell = (torch.eye(3) * L).reshape(1, 3, 3).contiguous().to(DEV)
    pbc = torch.ones(1, 3, dtype=torch.bool, device=DEV)
    ptr = torch.tensor([0, N], dtype=torch.int32, device=DEV)
    assert N * K * 3 > 2 ** 31
    nm, nn, sh, bidx = build_on_gpu(pos, cell, pbc, ptr, rc, K)
    assert int(nn.max()) < K
    assert abs(float(nn.float().mean()) - 4 / 3 * math.pi * rc ** 3 * rho) < 0.1
    # rows at both ends of the flat index range, and in between, against a search over all atoms
    sample = [0, 1, N // 2, N - 2, N - 1] + torch.randint(0, N, (20,), generator=g).tolist()
    rows_equal_brute_force(pos, cell[0], rc, nm, nn, sh, sample, 0, N)
    i, j, S = edge_list(nm, nn, sh)
    assert_symmetric(i, j, S, N)
    eps, sig = 0.01, 1.5  # random positions: keep the repulsive wall short
    e, f, w, es = gpu_lj(pos, cell, nm, sh, nn, bidx, eps, sig, rc, virial=True)
    # the same with the rows walked in the build's cell order (what the hook arranges for systems
    # this large): a permutation of the atoms, and identical per-atom results
    from nvalchemi_amd import _lib

    order = torch.empty(N, dtype=torch.int32, device=DEV)
    _lib.nl_atom_order(bidx, 1, order)
    assert torch.equal(order.long().sort().values, torch.arange(N, device=DEV))
    e2, f2 = torch.empty_like(e), torch.empty_like(f)
    es2 = torch.empty_like(es)
    _lib.lj_energy_forces(pos, cell, nm, sh, nn, bidx, N, eps, sig, rc, 0.0, False, e2, f2, None, es2, row_order=order)
    torch.cuda.synchronize()
    assert torch.equal(e2, e) and torch.equal(f2, f)
    assert abs(float(es2[0]) - float(es[0])) <= 1e-6 * abs(float(es[0]))
    e_sys, f64, w_tr, f_terms = torch_lj_over_edges(pos, cell, bidx, i, j, S, eps, sig, rc, 1)
    del i, j, S
    assert math.isfinite(float(es[0]))
    assert abs(float(es[0]) - float(e_sys[0])) <= 1e-5 * abs(float(e_sys[0]))
    assert abs(float(e.double().sum()) - float(e_sys[0])) <= 1e-5 * abs(float(e_sys[0]))
    tr = float(w.double()[0, 0] + w.double()[0, 4] + w.double()[0, 8])
    assert abs(tr - float(w_tr[0])) <= 1e-5 * abs(float(w_tr[0])) + 1e-6
    # uniform random positions put some atoms between close neighbors whose huge pair terms cancel:
    # beyond the bar, an atom is allowed the rounding of a float64 sum of its terms
    assert close(f, f64, slack=1e-13 * f_terms[:, None])
    # and the hinted call (shifts derived: this cell is far wider than twice the cutoff) is the same
    e3, f3 = torch.empty_like(e), torch.empty_like(f)
    _lib.lj_energy_forces(pos, cell, nm, sh, nn, bidx, N, eps, sig, rc, 0.0, False, e3, f3, None, es2, row_order=order,
                          neighbor_list_cutoff=rc)
    torch.cuda.synchronize()
    assert torch.equal(e3, e) and torch.equal(f3, f)
