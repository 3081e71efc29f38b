"""Host-side Tensor / SliceTensor / IndexMapping semantics through the C ABI (no device needed); expectations of
the reference's unittest/tensor/test_Tensor.cpp:14-150 and unittest/tensor/test_SliceTensor.cpp:12-100."""
import numpy as np
import pytest

import acrotensor_amd as at


def test_constructor_asserts():
    with pytest.raises(at.AcroError):
        at.Tensor()
    with pytest.raises(at.AcroError):
        at.Tensor(3, 0)
    with pytest.raises(at.AcroError):
        at.Tensor(-1)


def test_rank_dims_size_strides():
    T = at.Tensor(2, 3, 4)
    assert T.GetRank() == 3 and T.GetSize() == 24 and T.dims == (2, 3, 4)
    assert [T.GetStride(d) for d in range(3)] == [12, 4, 1]
    T9 = at.Tensor(1, 2, 1, 2, 1, 2, 1, 2, 3)
    assert T9.GetRank() == 9 and T9.GetSize() == 48
    T12 = at.Tensor(*([2] * 12))
    assert T12.GetRank() == 12 and T12.GetSize() == 4096


def test_row_major_index_coverage():
    T = at.Tensor(3, 4, 5)
    T.data[...] = np.arange(60.0).reshape(3, 4, 5)
    assert T.data[2, 1, 3] == 2 * 20 + 1 * 5 + 3
    flat = T.data.reshape(-1)
    assert np.array_equal(flat, np.arange(60.0))


def test_set_mult_on_host():
    T = at.Tensor(4, 4)
    T.Set(2.0)
    T.Mult(3.0)
    assert np.all(T.data == 6.0)


def test_reshape_keeps_data_and_checks_size():
    T = at.Tensor(4, 6)
    T.data[...] = np.arange(24.0).reshape(4, 6)
    T.Reshape(2, 3, 4)
    assert T.dims == (2, 3, 4) and np.array_equal(T.data.reshape(-1), np.arange(24.0))
    with pytest.raises(at.AcroError):
        T.Reshape(5, 5)


def test_external_host_buffer():
    buf = np.arange(6.0).reshape(2, 3).copy()
    T = at.Tensor(2, 3, hdata=buf)
    T.Mult(2.0)
    assert np.array_equal(buf, np.arange(6.0).reshape(2, 3) * 2)


def test_slices_alias_the_parent():
    T = at.Tensor(3, 4, 5)
    T.data[...] = np.arange(60.0).reshape(3, 4, 5)
    S = at.SliceTensor(T, 2)
    assert S.GetRank() == 2 and S.dims == (4, 5) and [S.GetStride(0), S.GetStride(1)] == [5, 1]
    assert np.array_equal(S.data, T.data[2])
    S2 = at.SliceTensor(T, 1, 3)
    assert S2.dims == (5,) and np.array_equal(S2.data, T.data[1, 3])
    S.Set(-1.0)
    assert np.all(T.data[2] == -1.0) and np.all(T.data[:2] >= 0)
    with pytest.raises(at.AcroError):
        at.SliceTensor(T, 0, 0, 0)           # cannot slice away every dimension
    with pytest.raises(at.AcroError):
        at.SliceTensor(T, 5)


def test_index_mapping_inverse_is_a_stable_compressed_row_form(checker):
    M = at.IndexMapping(4, 8)
    M.map[:] = [3, 1, 2, 3, 0, 1, 1, 2]
    with pytest.raises(at.AcroError):
        M.inverse
    M.ComputeInverse()
    inv, off = M.inverse
    assert list(inv) == [4, 1, 5, 6, 2, 7, 0, 3] and list(off) == [0, 1, 4, 6, 8]
    oinv, ooff = checker.index_mapping_inverse(M.map, 4)      # same as the reference when every entry has a preimage
    assert np.array_equal(inv, oinv) and np.array_equal(off, ooff)
    with pytest.raises(at.AcroError):
        M.ComputeInverse()


def test_index_mapping_rows_stay_aligned_when_domain_entries_have_no_preimage():
    M = at.IndexMapping(5, 4)
    M.map[:] = [4, 0, 4, 2]
    M.ComputeInverse()
    inv, off = M.inverse
    assert list(off) == [0, 1, 1, 2, 2, 4] and list(inv) == [1, 3, 0, 2]
