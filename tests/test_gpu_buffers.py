"""HIP masked copy / compaction kernels against the numpy oracle, through the package's mirror of
nvalchemi/data/buffer_kernels.py: the reference's own cases (test/data/test_buffer_kernels.py),
random inputs in every supported dtype and row size (16-, 4- and 1-byte copy units), sizes beyond
one scan block, and conservation of every row at a size the oracle does not see."""

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.float64, torch.int32, torch.int64, torch.bool]


def T(a):
    return torch.as_tensor(np.ascontiguousarray(a), device=DEV)


def N(t):
    return t.cpu().numpy()


def random_rows(rng, shape, dtype):
    if dtype == torch.bool:
        return rng.random(shape) < 0.5
    a = rng.integers(1, 1 << 20, shape)
    return a.astype({torch.float32: np.float32, torch.float64: np.float64, torch.int32: np.int32,
                     torch.int64: np.int64}[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols", [1, 3, 4, 9, 16])
def test_rows_put_fit_defrag_match_oracle(dtype, cols):
    from nvalchemi_amd.data import buffer_kernels as bk

    rng = np.random.default_rng(cols)
    for n_src, n_dest, p_mask, p_full in [(6, 6, 0.6, 0.0), (5, 4, 0.8, 0.5), (700, 300, 0.5, 0.3),
                                          (2500, 4000, 0.4, 0.6), (3, 0, 1.0, 0.0)]:
        src = random_rows(rng, (n_src, cols), dtype)
        mask = rng.random(n_src) < p_mask
        # occupied slots first, then the empty tail: the layout the callers keep
        n_full = int(n_dest * p_full)
        dmask = np.arange(n_dest) < n_full
        dest = np.where(dmask[:, None], random_rows(rng, (n_dest, cols), dtype), np.zeros((n_dest, cols), src.dtype))
        copied = np.zeros(n_src, bool)
        fit = np.zeros(n_src, bool)
        g_src, g_mask, g_dest, g_dmask, g_copied, g_fit = T(src), T(mask), T(dest), T(dmask), T(copied), T(fit)
        bk.compute_put_fit_mask_per_system(g_mask, g_dmask, g_fit)
        oracle.put_fit_mask_per_system(mask, dmask, fit)
        assert np.array_equal(N(g_fit), fit)
        bk.put_masked_per_system(g_src, g_mask, g_dest, g_dmask, g_copied)
        oracle.put_masked_per_system(src, mask, dest, dmask, copied)
        assert np.array_equal(N(g_dest), dest) and np.array_equal(N(g_dmask), dmask)
        assert np.array_equal(N(g_copied), copied) and np.array_equal(copied, fit)
        bk.defrag_per_system(g_src, g_copied)
        oracle.defrag_per_system(src, copied)
        assert np.array_equal(N(g_src), src) and np.array_equal(N(g_copied), copied)


def test_rows_scattered_empty_slots_follow_the_reference():
    """Empty slots that are not a tail: rows still go to consecutive slots from the first empty one
    (nvalchemi/data/buffer_kernels.py:183), over an occupied slot if one is in the way."""
    from nvalchemi_amd.data import buffer_kernels as bk

    src = np.arange(8, dtype=np.float32).reshape(4, 2) + 1
    mask = np.array([True, True, False, True])
    dmask = np.array([True, False, True, False, False])
    dest = np.full((5, 2), -1, np.float32)
    copied = np.zeros(4, bool)
    g = [T(src), T(mask), T(dest), T(dmask), T(copied)]
    bk.put_masked_per_system(*g)
    oracle.put_masked_per_system(src, mask, dest, dmask, copied)
    assert np.array_equal(N(g[2]), dest) and np.array_equal(N(g[3]), dmask) and np.array_equal(N(g[4]), copied)
    assert copied.sum() == 3 and np.array_equal(dest[1:4], src[mask])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("elem", [(1,), (3,), (4,), (3, 3)])
def test_segments_put_fit_defrag_match_oracle(dtype, elem):
    from nvalchemi_amd.data import buffer_kernels as bk

    rng = np.random.default_rng(len(elem) * 7 + elem[0])
    for n, max_len, cap_frac, n_dest0 in [(3, 4, 2.0, 0), (12, 6, 0.5, 2), (300, 40, 0.7, 5), (2100, 9, 0.6, 0),
                                          (5, 0, 1.0, 0)]:
        lengths = rng.integers(0, max_len + 1, n)
        ptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        total = int(ptr[-1])
        src = random_rows(rng, (total,) + elem, dtype)
        mask = rng.random(n) < 0.6
        # destination with n_dest0 segments already in it
        lens0 = rng.integers(1, 5, n_dest0)
        used = int(lens0.sum())
        cap = used + int(cap_frac * total)
        dptr = np.zeros(n_dest0 + n + 2 + 3, np.int32)
        dptr[: n_dest0 + 1] = np.concatenate([[0], np.cumsum(lens0)])
        dest = np.zeros((cap, int(np.prod(elem))), src.dtype)
        dest[:used] = random_rows(rng, (used, int(np.prod(elem))), dtype)
        copied, fit = np.zeros(n, bool), np.zeros(n, bool)
        g_src, g_ptr, g_mask, g_dest, g_dptr, g_copied, g_fit = (T(src), T(ptr), T(mask), T(dest), T(dptr), T(copied),
                                                                 T(fit))
        bk.compute_put_fit_mask_segmented(g_ptr, g_mask, g_dptr, n_dest0, cap, g_fit)
        oracle.put_fit_mask_segmented(ptr, mask, dptr, n_dest0, cap, fit)
        assert np.array_equal(N(g_fit), fit)
        new = bk.put_masked_segmented(g_src, g_ptr, g_mask, g_dest, g_dptr, n_dest0, g_copied)
        want = oracle.put_masked_segmented(src, ptr, mask, dest, dptr, n_dest0, copied)
        assert int(new[0]) == want and np.array_equal(copied, fit)
        assert np.array_equal(N(g_dest), dest) and np.array_equal(N(g_dptr), dptr) and np.array_equal(N(g_copied), copied)
        kept = bk.defrag_segmented(g_src, g_ptr, g_copied)
        assert int(kept[0]) == oracle.defrag_segmented(src, ptr, copied)
        assert np.array_equal(N(g_src), src) and np.array_equal(N(g_ptr), ptr)


def test_segments_edge_cases_of_the_reference():
    from nvalchemi_amd.data import buffer_kernels as bk

    # no systems: defrag writes a zero boundary and returns 0; put returns None
    ptr = torch.tensor([7], dtype=torch.int32, device=DEV)
    src = torch.zeros(0, 2, device=DEV)
    kept = bk.defrag_segmented(src, ptr, torch.zeros(0, dtype=torch.bool, device=DEV))
    assert int(kept[0]) == 0 and int(ptr[0]) == 0
    assert bk.put_masked_segmented(src, ptr, torch.zeros(0, dtype=torch.bool, device=DEV), torch.zeros(4, 2, device=DEV),
                                   torch.zeros(4, dtype=torch.int32, device=DEV), 0,
                                   torch.zeros(0, dtype=torch.bool, device=DEV)) is None
    # a destination pointer without room for new boundaries: ValueError from put, cleared mask from fit
    sptr = torch.tensor([0, 2, 3], dtype=torch.int32, device=DEV)
    ones = torch.ones(2, dtype=torch.bool, device=DEV)
    short = torch.tensor([0, 10], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError):
        bk.put_masked_segmented(torch.zeros(3, 2, device=DEV), sptr, ones, torch.zeros(100, 2, device=DEV), short, 1,
                                torch.zeros(2, dtype=torch.bool, device=DEV))
    fit = torch.ones(2, dtype=torch.bool, device=DEV)
    bk.compute_put_fit_mask_segmented(sptr, ones, short, 1, 100, fit)
    assert not bool(fit.any())
    # an int64 boundary tensor is accepted by defrag and written back
    ptr64 = torch.tensor([0, 1, 3], dtype=torch.int64, device=DEV)
    data = torch.arange(3, dtype=torch.float32, device=DEV).view(3, 1)
    kept = bk.defrag_segmented(data, ptr64, torch.tensor([True, False], device=DEV))
    assert int(kept[0]) == 1 and ptr64.tolist() == [0, 2, 2] and data.view(-1).tolist() == [1.0, 2.0, 0.0]
    # a source buffer longer than its last segment: the rows behind it are neither moved nor kept
    ptr = torch.tensor([0, 2, 4], dtype=torch.int32, device=DEV)
    data = torch.arange(1, 9, dtype=torch.int32, device=DEV).view(8, 1)
    kept = bk.defrag_segmented(data, ptr, torch.tensor([True, False], device=DEV))
    assert int(kept[0]) == 1 and ptr.tolist() == [0, 2, 2] and data.view(-1).tolist() == [3, 4, 0, 0, 0, 0, 0, 0]
    # unsupported dtype, as in the reference's dtype table
    with pytest.raises(KeyError):
        bk.defrag_per_system(torch.zeros(4, 2, dtype=torch.float16, device=DEV),
                             torch.zeros(4, dtype=torch.bool, device=DEV))


def test_large_refill_round_trip_conserves_rows():
    """256 systems x ~3900 atoms of float32 positions: finished systems leave for a second buffer,
    the rest is compacted; every system's rows arrive intact (checked on the device, by segment sums
    and a full comparison of gathered rows)."""
    from nvalchemi_amd.data import buffer_kernels as bk

    g = torch.Generator().manual_seed(3)
    n = 256
    lengths = torch.randint(3700, 4100, (n,), generator=g)
    ptr = torch.cat([torch.zeros(1, dtype=torch.long), lengths.cumsum(0)]).to(torch.int32).to(DEV)
    total = int(ptr[-1])
    src = torch.rand(total, 3, generator=g).to(DEV)
    orig, optr = src.clone(), ptr.clone()
    mask = (torch.rand(n, generator=g) < 0.4).to(DEV)
    dest = torch.zeros(total // 3, 3, device=DEV)  # not everything fits
    dptr = torch.zeros(n + 2, dtype=torch.int32, device=DEV)
    copied = torch.zeros(n, dtype=torch.bool, device=DEV)
    new = int(bk.put_masked_segmented(src, ptr, mask, dest, dptr, 0, copied)[0])
    assert 0 < new == int(copied.sum()) < int(mask.sum())
    moved = torch.nonzero(copied).view(-1).tolist()
    for k, i in enumerate(moved):
        assert torch.equal(dest[int(dptr[k]): int(dptr[k + 1])], orig[int(optr[i]): int(optr[i + 1])])
    kept = int(bk.defrag_segmented(src, ptr, copied)[0])
    stay = torch.nonzero(~copied).view(-1).tolist()
    assert kept == len(stay)
    for k, i in enumerate(stay):
        assert torch.equal(src[int(ptr[k]): int(ptr[k + 1])], orig[int(optr[i]): int(optr[i + 1])])
    assert not bool(src[int(ptr[kept]):].any()) and int(ptr[-1]) == int(ptr[kept])
