"""Pins the numpy restatement of the neighbor filters with the reference's own cases
(test/models/test_neighbor_filter.py:49-760: the 4-atom chain, the image pair through a 5 A cell,
per-system cells, shift bookkeeping, COO variants, matrix -> list), restated with the same inputs
and expected results.  CPU only."""

import numpy as np
import pytest

import oracle


def chain():
    pos = np.array([[0.0, 0, 0], [1.0, 0, 0], [3.0, 0, 0], [5.0, 0, 0]], dtype=np.float32)
    nm = np.array([[1, 2, 4], [0, 2, 4], [0, 1, 4], [4, 4, 4]], dtype=np.int32)
    nn = np.array([2, 2, 2, 0], dtype=np.int32)
    return pos, nm, nn, 4


def chain_coo():
    pos = chain()[0]
    nl = np.array([[0, 1], [0, 2], [1, 0], [1, 2], [2, 0], [2, 1]], dtype=np.int32)
    return pos, nl, np.array([0, 2, 4, 6, 6], dtype=np.int32)


def test_matrix_filter_on_the_chain():
    pos, nm, nn, fill = chain()
    out, cnt, sh = oracle.filter_neighbor_matrix(pos, 1.5, nm, nn, fill)
    assert list(cnt) == [1, 1, 0, 0] and out[0, 0] == 1 and out[1, 0] == 0 and sh is None
    out, cnt, _ = oracle.filter_neighbor_matrix(pos, 2.5, nm, nn, fill)
    assert list(cnt) == [1, 2, 1, 0]
    for i in range(4):  # survivors first, padding behind
        assert (out[i, : cnt[i]] < fill).all() and (out[i, cnt[i]:] == fill).all()
    assert out[2, 0] == 1  # the survivor of row 2 moved to the front
    out, cnt, _ = oracle.filter_neighbor_matrix(pos, 10.0, nm, nn, fill)
    assert np.array_equal(out, nm) and np.array_equal(cnt, nn)
    out, cnt, _ = oracle.filter_neighbor_matrix(pos, 0.1, nm, nn, fill)
    assert (out == fill).all() and not cnt.any()
    assert cnt.dtype == nn.dtype and out.shape == nm.shape


def test_matrix_filter_with_images_and_per_system_cells():
    pos = np.array([[0.0, 0, 0], [4.5, 0, 0]], dtype=np.float32)
    nm = np.array([[1, 2], [0, 2]], dtype=np.int32)
    sh = np.array([[[-1, 0, 0], [0, 0, 0]], [[1, 0, 0], [0, 0, 0]]], dtype=np.int32)
    _, cnt, out_sh = oracle.filter_neighbor_matrix(pos, 2.0, nm, np.array([1, 1], np.int32), 2,
                                                   cell=5.0 * np.eye(3, dtype=np.float32), neighbor_matrix_shifts=sh)
    assert list(cnt) == [1, 1] and np.array_equal(out_sh, sh)
    # without the cell the direct distance 4.5 decides
    _, cnt, _ = oracle.filter_neighbor_matrix(pos, 2.0, nm, np.array([1, 1], np.int32), 2, neighbor_matrix_shifts=sh)
    assert list(cnt) == [0, 0]
    pos = np.array([[0.0, 0, 0], [4.5, 0, 0], [0.0, 0, 0], [1.0, 0, 0]], dtype=np.float32)
    cells = np.stack([5.0 * np.eye(3), 10.0 * np.eye(3)]).astype(np.float32)
    nm = np.array([[1, 4], [0, 4], [3, 4], [2, 4]], dtype=np.int32)
    sh = np.zeros((4, 2, 3), np.int32)
    sh[0, 0], sh[1, 0] = [-1, 0, 0], [1, 0, 0]
    _, cnt, _ = oracle.filter_neighbor_matrix(pos, 2.0, nm, np.ones(4, np.int32), 4, cell=cells,
                                              neighbor_matrix_shifts=sh, batch_idx=np.array([0, 0, 1, 1], np.int32))
    assert list(cnt) == [1, 1, 1, 1]
    with pytest.raises(ValueError):
        oracle.filter_neighbor_matrix(pos, 2.0, nm, np.ones(4, np.int32), 4, cell=cells, neighbor_matrix_shifts=sh)


def test_matrix_filter_carries_shifts_with_their_entries():
    pos, nm, nn, fill = chain()
    sh = np.zeros((4, 3, 3), np.int32)
    for i in range(4):
        for k in range(3):
            sh[i, k, 0] = i * 10 + k
    out, cnt, out_sh = oracle.filter_neighbor_matrix(pos, 2.5, nm, nn, fill, neighbor_matrix_shifts=sh)
    where = {(i, int(nm[i, k])): k for i in range(4) for k in range(3) if nm[i, k] < fill}
    for i in range(4):
        for k in range(cnt[i]):
            assert np.array_equal(out_sh[i, k], sh[i, where[(i, int(out[i, k]))]])
        assert not out_sh[i, cnt[i]:].any()


def test_list_filter_on_the_chain():
    pos, nl, ptr = chain_coo()
    out, optr, sh = oracle.filter_neighbor_list(pos, 1.5, nl, ptr)
    assert out.tolist() == [[0, 1], [1, 0]] and optr.tolist() == [0, 1, 2, 2, 2] and sh is None
    out, optr, _ = oracle.filter_neighbor_list(pos, 2.5, nl, ptr)
    assert out.tolist() == [[0, 1], [1, 0], [1, 2], [2, 1]] and optr.tolist() == [0, 1, 3, 4, 4]
    out, optr, _ = oracle.filter_neighbor_list(pos, 0.1, nl, ptr)
    assert out.shape == (0, 2) and not optr.any()
    out, optr, _ = oracle.filter_neighbor_list(pos, 10.0, nl, ptr)
    assert np.array_equal(out, nl) and np.array_equal(optr, ptr)
    # the image pair
    pos = np.array([[0.0, 0, 0], [4.5, 0, 0]], dtype=np.float32)
    nl = np.array([[0, 1], [1, 0]], dtype=np.int32)
    sh = np.array([[-1, 0, 0], [1, 0, 0]], dtype=np.int32)
    out, optr, osh = oracle.filter_neighbor_list(pos, 2.0, nl, np.array([0, 1, 2], np.int32),
                                                 cell=5.0 * np.eye(3, dtype=np.float32), neighbor_list_shifts=sh)
    assert len(out) == 2 and np.array_equal(osh, sh) and optr.tolist() == [0, 1, 2]


def test_matrix_to_list():
    pos, nm, nn, fill = chain()
    nl, ptr, sh = oracle.neighbor_matrix_to_list(nm, nn, fill)
    assert nl.tolist() == [[0, 1], [0, 2], [1, 0], [1, 2], [2, 0], [2, 1]] and ptr.tolist() == [0, 2, 4, 6, 6]
    assert sh is None and nl.dtype == np.int32 and ptr.dtype == np.int32
    shifts = np.arange(36, dtype=np.int32).reshape(4, 3, 3)
    nl, ptr, sh = oracle.neighbor_matrix_to_list(nm, nn, fill, shifts)
    assert sh.shape == (6, 3) and np.array_equal(sh[1], shifts[0, 1]) and np.array_equal(sh[5], shifts[2, 1])
    nm2 = np.array([[1, 2, 3], [0, 4, 4], [4, 4, 4], [0, 1, 4]], dtype=np.int32)
    nl, ptr, _ = oracle.neighbor_matrix_to_list(nm2, np.array([3, 1, 0, 2], np.int32), 4)
    assert ptr.tolist() == [0, 3, 4, 4, 6] and len(nl) == 6
