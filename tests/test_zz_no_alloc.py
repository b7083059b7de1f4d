"""The entry point that allocates nothing (``nvamd_lj_energy_forces_static``: the pair kernel's
scratch in a device array built into the library) against the entry point it is a variant of
(``nvamd_lj_energy_forces_hinted`` with a caller's workspace), through the C ABI: same per-atom
energies and forces bit for bit, per-system energies and virials within 1e-5 relative / 1e-6 absolute
(their float64 atomics arrive in a different order from call to call), on two calls in a row, the
second with a smaller input (fewer atoms and systems), so that what the first call left in the shared
array must not leak into the second."""

import numpy as np
import pytest
import torch

import oracle
from _systems import sheared_fcc_boxes

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(seed, n_boxes, reps):
    P, C, pb, ptr = sheared_fcc_boxes(seed=seed, n_boxes=n_boxes, reps=reps)
    rc = 2.5
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc, 96)
    assert nn.max() < 96
    bi = oracle.batch_idx_from_ptr(ptr)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)  # noqa: E731
    return dict(pos=t(P), cells=t(C), nm=t(nm), sh=t(sh), nn=t(nn), bi=t(bi), N=len(P), B=len(ptr) - 1, rc=rc,
                ref=oracle.lj_matrix(P, C, nm, sh, nn, bi, len(P), 1.0, 1.0, rc, virial=True))


def _run(fn, c, **kw):
    N, B = c["N"], c["B"]
    out = dict(e=torch.full((N,), 7.0, device=DEV), f=torch.full((N, 3), 7.0, device=DEV),
               w=torch.full((B, 9), 7.0, device=DEV), es=torch.full((B,), 7.0, device=DEV))
    fn(c["pos"], c["cells"], c["nm"], c["sh"], c["nn"], c["bi"], N, 1.0, 1.0, c["rc"], 0.0, **kw,
       atomic_energies=out["e"], forces=out["f"], virials=out["w"], system_energies=out["es"])
    torch.cuda.synchronize()
    return {k: v.cpu().numpy() for k, v in out.items()}


def test_static_scratch_entry_matches_the_workspace_entry_on_two_calls_in_a_row():
    from nvalchemi_amd import _lib

    big, small = _case(11, 6, 4), _case(12, 2, 3)
    assert small["N"] < big["N"] and small["B"] < big["B"]
    for c in (big, small):
        want = _run(_lib.lj_energy_forces, c, half_list=False)
        got = _run(_lib.lj_energy_forces_static, c)
        assert np.array_equal(got["e"], want["e"]) and np.array_equal(got["f"], want["f"])
        for k in ("es", "w"):
            assert np.all(np.abs(got[k] - want[k]) <= 1e-6 + 1e-5 * np.abs(want[k])), k
        # and both against the oracle
        ref = c["ref"]
        assert np.all(np.abs(got["f"] - ref["forces"]) <= 1e-6 + 1e-5 * np.abs(ref["forces"]))
        assert np.all(np.abs(got["es"] - ref["energy"]) <= 1e-6 + 1e-5 * np.abs(ref["energy"]))
        assert np.all(np.abs(got["w"] - ref["virials"]) <= 1e-5 + 1e-5 * np.abs(ref["virials"]))


def test_static_scratch_entry_takes_no_device_memory():
    """What the entry point is named for: between two calls the free device memory does not move (the outputs
    are allocated beforehand; the first call on the device, which looks up the array's address, came earlier)."""
    from nvalchemi_amd import _lib

    c = _case(13, 3, 3)
    N, B = c["N"], c["B"]
    out = dict(e=torch.empty(N, device=DEV), f=torch.empty(N, 3, device=DEV), w=torch.empty(B, 9, device=DEV),
               es=torch.empty(B, device=DEV))

    def call():
        _lib.lj_energy_forces_static(c["pos"], c["cells"], c["nm"], c["sh"], c["nn"], c["bi"], N, 1.0, 1.0, c["rc"], 0.0,
                                     atomic_energies=out["e"], forces=out["f"], virials=out["w"], system_energies=out["es"])
        torch.cuda.synchronize()

    call()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before and torch.cuda.memory_reserved() == reserved_before


def test_static_scratch_entry_at_its_largest_number_of_systems():
    """16 384 systems of two atoms each, the most the built-in scratch holds: same results as the workspace entry."""
    from nvalchemi_amd import _lib

    B = _lib.LJ_STATIC_MAX_SYSTEMS
    N = 2 * B
    g = torch.Generator().manual_seed(5)
    first = torch.rand(B, 3, generator=g) * 5.0 + 2.0
    bond = torch.nn.functional.normalize(torch.randn(B, 3, generator=g), dim=1) * (1.0 + torch.rand(B, 1, generator=g))
    pos = torch.stack([first, first + bond], 1).reshape(N, 3).to(DEV)
    cells = (torch.eye(3) * 12.0).repeat(B, 1, 1).to(DEV)
    partner = torch.arange(N, dtype=torch.int32).reshape(B, 2).flip(1).reshape(N, 1)
    nm = torch.cat([partner, torch.full((N, 3), N, dtype=torch.int32)], 1).contiguous().to(DEV)
    c = dict(pos=pos, cells=cells, nm=nm, sh=torch.zeros(N, 4, 3, dtype=torch.int32, device=DEV),
             nn=torch.ones(N, dtype=torch.int32, device=DEV),
             bi=torch.arange(B, dtype=torch.int32).repeat_interleave(2).to(DEV), N=N, B=B, rc=2.5)
    want = _run(_lib.lj_energy_forces, c, half_list=False)
    got = _run(_lib.lj_energy_forces_static, c)
    assert np.array_equal(got["e"], want["e"]) and np.array_equal(got["f"], want["f"])
    for k in ("es", "w"):
        assert np.all(np.abs(got[k] - want[k]) <= 1e-6 + 1e-5 * np.abs(want[k])), k
    # a dimer's energy is the pair energy, half of it on each atom
    p64 = pos.cpu().double().reshape(B, 2, 3)  # (the float32 positions the kernel saw)
    r = (p64[:, 1] - p64[:, 0]).norm(dim=1).numpy()
    u = 4.0 * (r ** -12 - r ** -6)
    assert np.allclose(got["es"], u, rtol=1e-5, atol=1e-6)


def test_static_scratch_entry_rejects_more_systems_than_it_holds():
    from nvalchemi_amd import _lib

    B = _lib.LJ_STATIC_MAX_SYSTEMS + 1
    z = lambda *s, dt=torch.float32: torch.zeros(*s, dtype=dt, device=DEV)  # noqa: E731
    with pytest.raises(_lib.KernelLibraryError, match="at most"):
        _lib.lj_energy_forces_static(z(4, 3), z(B, 3, 3), z(4, 4, dt=torch.int32), None, z(4, dt=torch.int32),
                                     z(4, dt=torch.int32), 4, 1.0, 1.0, 2.5, 0.0, z(4), z(4, 3), None, z(B))
