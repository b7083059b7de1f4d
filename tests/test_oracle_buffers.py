"""Pins the numpy restatement of the masked copy / compaction functions with the reference's own
cases (test/data/test_buffer_kernels.py:49-535, restated: same inputs, same expected results) and
with brute-force properties on random inputs.  CPU only."""

import numpy as np
import pytest

import oracle

DTYPES = [np.float32, np.float64, np.int32, np.int64, np.bool_]


def arange(shape, dtype):
    a = np.arange(int(np.prod(shape)))
    return (a % 2 == 1 if dtype is np.bool_ else a).astype(dtype).reshape(shape)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rows_enough_room(dtype):
    src = arange((6, 2), dtype)
    mask = np.array([True, False, True, False, True, True])
    copied = np.zeros(6, bool)
    dest, dmask = np.zeros((6, 2), dtype), np.zeros(6, bool)
    oracle.put_masked_per_system(src, mask, dest, dmask, copied)
    assert copied.sum() == 4 and dmask.sum() == 4
    assert np.array_equal(dest[dmask], src[mask])
    assert np.array_equal(dmask, [True] * 4 + [False] * 2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rows_not_enough_room(dtype):
    src = arange((5, 2), dtype)
    mask = np.array([True, True, True, False, True])
    copied = np.zeros(5, bool)
    dest, dmask = np.zeros((4, 2), dtype), np.array([False, False, True, True])
    oracle.put_masked_per_system(src, mask, dest, dmask, copied)
    assert list(copied) == [True, True, False, False, False] and dmask.all()
    assert np.array_equal(dest[:2], src[:2])
    fit = np.zeros(5, bool)
    oracle.put_fit_mask_per_system(mask, np.array([False, False, True, True]), fit)
    assert list(fit) == [True, True, False, False, False]


def test_rows_fit_mask_enough_room_and_views_and_empties():
    fit = np.zeros(5, bool)
    oracle.put_fit_mask_per_system(np.array([True, False, True, True, False]), np.zeros(10, bool), fit)
    assert list(fit) == [True, False, True, True, False]
    for shape in [(6, 1), (4, 3, 3)]:
        src = arange(shape, np.float32)
        n = shape[0]
        dest, dmask, copied = np.zeros((n, src.size // n), np.float32), np.zeros(n, bool), np.zeros(n, bool)
        oracle.put_masked_per_system(src, np.ones(n, bool), dest, dmask, copied)
        assert np.array_equal(dest, src.reshape(n, -1)) and copied.all()
    # no masked rows, and an empty source: nothing changes
    dest, dmask, copied = np.zeros((4, 2), np.float32), np.zeros(4, bool), np.zeros(4, bool)
    oracle.put_masked_per_system(arange((4, 2), np.float32), np.zeros(4, bool), dest, dmask, copied)
    assert not copied.any() and not dmask.any() and not dest.any()
    oracle.put_masked_per_system(np.zeros((0, 2), np.float32), np.zeros(0, bool), dest, dmask, np.zeros(0, bool))
    assert not dmask.any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_rows_defrag_tail_zeros(dtype):
    src = arange((6, 2), dtype)
    orig = src.copy()
    mask = np.array([True, False, True, False, True, False])
    copied = np.zeros(6, bool)
    oracle.put_masked_per_system(src, mask, np.zeros((6, 2), dtype), np.zeros(6, bool), copied)
    oracle.defrag_per_system(src, copied)
    assert (~copied).sum() == 3 and list(copied) == [False] * 3 + [True] * 3
    assert np.array_equal(src[:3], orig[~mask]) and not src[3:].any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_segments_put(dtype):
    ptr = np.array([0, 2, 5, 6], np.int32)
    src = arange((6, 2), dtype)
    copied = np.zeros(3, bool)
    dest, dptr = np.zeros((10, 2), dtype), np.zeros(5, np.int32)
    new = oracle.put_masked_segmented(src, ptr, np.array([True, False, True]), dest, dptr, 0, copied)
    assert new == 2 and list(dptr[:3]) == [0, 2, 3] and list(copied) == [True, False, True]
    assert np.array_equal(dest[0:2], src[0:2]) and np.array_equal(dest[2:3], src[5:6])
    assert dptr[3] == 3  # one more copy of the last end (buffer_kernels.py:657-658)
    # element shapes (2,) and (3, 3)
    for elem in [(2,), (3, 3)]:
        src = arange((3,) + elem, dtype)
        dest, dptr = np.zeros((10, int(np.prod(elem))), dtype), np.zeros(5, np.int32)
        new = oracle.put_masked_segmented(src, np.array([0, 1, 3], np.int32), np.ones(2, bool), dest, dptr, 0,
                                          np.zeros(2, bool))
        assert new == 2 and list(dptr[:3]) == [0, 1, 3] and np.array_equal(dest[:3], src.reshape(3, -1))
    with pytest.raises(ValueError):
        oracle.put_masked_segmented(src, np.array([0, 1, 3], np.int32), np.ones(2, bool), dest,
                                    np.zeros(3, np.int32), 0, np.zeros(2, bool))


def test_segments_fit_masks():
    fit = np.zeros(3, bool)
    oracle.put_fit_mask_segmented(np.array([0, 2, 3, 6], np.int32), np.array([True, False, True]),
                                  np.array([0, 5, 5, 5, 5, 5], np.int32), 1, 20, fit)
    assert list(fit) == [True, False, True]
    fit = np.ones(2, bool)  # no room for new boundaries: cleared
    oracle.put_fit_mask_segmented(np.array([0, 2, 3], np.int32), np.ones(2, bool), np.array([0, 10], np.int32),
                                  1, 100, fit)
    assert not fit.any()
    fit = np.zeros(2, bool)  # 4 rows free: the 2-row segment fits, the 5-row one behind it does not
    oracle.put_fit_mask_segmented(np.array([0, 2, 7], np.int32), np.ones(2, bool), np.zeros(6, np.int32), 0, 4, fit)
    assert list(fit) == [True, False]


@pytest.mark.parametrize("dtype", DTYPES)
def test_segments_defrag(dtype):
    ptr = np.array([0, 2, 5, 7], np.int32)
    src = arange((7, 2), dtype)
    orig = src.copy()
    assert oracle.defrag_segmented(src, ptr, np.array([False, True, False])) == 2
    assert ptr[0] == 0 and ptr[2] == 4 and not src[4:].any()
    assert np.array_equal(src[:4], np.concatenate([orig[0:2], orig[5:7]]))
    # lengths 0, 3, 1, 2; keep segments 1 and 3
    ptr = np.array([0, 0, 3, 4, 6], np.int32)
    src = arange((6, 1), dtype)
    orig = src.copy()
    assert oracle.defrag_segmented(src, ptr, np.array([True, False, True, False])) == 2
    assert list(ptr[:3]) == [0, 3, 5] and list(ptr[3:]) == [5, 5]
    assert np.array_equal(src[:3], orig[0:3]) and np.array_equal(src[3:5], orig[4:6]) and not src[5:].any()
    # keep the second of two, the middle of three
    ptr, src = np.array([0, 1, 3], np.int32), arange((3, 1), dtype)
    orig = src.copy()
    assert oracle.defrag_segmented(src, ptr, np.array([True, False])) == 1
    assert list(ptr[:2]) == [0, 2] and np.array_equal(src[:2], orig[1:3])
    ptr, src = np.array([0, 2, 5, 6], np.int32), arange((6, 1), dtype)
    orig = src.copy()
    assert oracle.defrag_segmented(src, ptr, np.array([True, False, True])) == 1
    assert list(ptr[:2]) == [0, 3] and np.array_equal(src[:3], orig[2:5])
    # no systems
    ptr = np.array([7], np.int32)
    assert oracle.defrag_segmented(np.zeros((0, 2), dtype), ptr, np.zeros(0, bool)) == 0 and ptr[0] == 0


def test_put_then_defrag_conserves_every_segment():
    """Random round trip: what left the source arrived in the destination, in order, and what
    stayed is compacted in order; nothing is duplicated or lost."""
    rng = np.random.default_rng(5)
    for _ in range(20):
        n = int(rng.integers(1, 12))
        lengths = rng.integers(0, 6, n)
        ptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        src = rng.integers(1, 1000, (int(ptr[-1]), 3)).astype(np.int64)
        orig, optr = src.copy(), ptr.copy()
        mask = rng.random(n) < 0.6
        cap = int(rng.integers(0, ptr[-1] + 3))
        dest, dptr = np.zeros((cap, 3), np.int64), np.zeros(n + 2, np.int32)
        copied = np.zeros(n, bool)
        new = oracle.put_masked_segmented(src, ptr, mask, dest, dptr, 0, copied)
        assert (copied <= mask).all() and new == copied.sum()
        moved = [orig[optr[i]: optr[i + 1]] for i in range(n) if copied[i]]
        got = [dest[dptr[k]: dptr[k + 1]] for k in range(new)]
        assert all(np.array_equal(a, b) for a, b in zip(moved, got))
        # the first masked segment that does not fit stops everything behind it
        laid = np.cumsum(np.where(mask, lengths, 0))
        assert np.array_equal(copied, mask & (laid <= cap))
        kept = oracle.defrag_segmented(src, ptr, copied)
        stay = [orig[optr[i]: optr[i + 1]] for i in range(n) if not copied[i]]
        assert kept == len(stay)
        assert all(np.array_equal(src[ptr[k]: ptr[k + 1]], s) for k, s in enumerate(stay))
        assert not src[ptr[kept]:].any()
