"""Tensor / SliceTensor / IndexMapping residency semantics on the device, as the reference tests them in
unittest/tensor/test_Tensor.cpp:155-184 and unittest/tensor/test_SliceTensor.cpp:105-168."""
import numpy as np
import pytest

from gpu_helpers import to_tensor

pytestmark = pytest.mark.gpu


def test_map_switch_set_move(at):
    T = at.Tensor(10, 10)
    T.Set(3.0)
    assert not T.IsMappedToGPU() and not T.IsOnGPU() and T.GetDeviceData() is None
    T.MapToGPU()
    assert T.IsMappedToGPU() and not T.IsOnGPU() and T.GetDeviceData()
    with pytest.raises(at.AcroError):
        T.MapToGPU()                                     # mapping twice
    T.SwitchToGPU()
    assert T.IsOnGPU()
    T.Set(9.0)                                           # on the device only
    assert np.all(T.data == 3.0)
    T.MoveFromGPU()
    assert not T.IsOnGPU() and np.all(T.data == 9.0)
    T.Set(2.0)
    T.MoveToGPU()
    T.Mult(2.5)
    assert np.all(T.data == 2.0)
    T.SwitchFromGPU()                                    # drop the device result
    assert np.all(T.data == 2.0)
    T.SwitchToGPU()
    T.MoveFromGPU()
    assert np.all(T.data == 5.0)
    T.UnmapFromGPU()
    assert not T.IsMappedToGPU() and not T.IsOnGPU()
    with pytest.raises(at.AcroError):
        T.UnmapFromGPU()


def test_move_to_gpu_maps_on_demand_and_is_idempotent(at):
    T = to_tensor(at, np.arange(12.0).reshape(3, 4))
    T.MoveToGPU()
    T.data[...] = -1.0                                   # host copy is stale now
    T.MoveToGPU()                                        # no copy: the device copy is current
    T.MoveFromGPU()
    assert np.array_equal(T.data, np.arange(12.0).reshape(3, 4))


def test_slices_share_storage_and_residency(at):
    T = to_tensor(at, np.zeros((3, 4, 5)))
    S1, S12 = at.SliceTensor(T, 1), at.SliceTensor(T, 1, 2)
    assert S1.dims == (4, 5) and S12.dims == (5,)
    S1.MoveToGPU()
    assert T.IsOnGPU() and S12.IsOnGPU() and T.IsMappedToGPU()
    S1.Set(4.0)
    S12.Set(7.0)
    T.MoveFromGPU()
    assert not S1.IsOnGPU()
    expected = np.zeros((3, 4, 5))
    expected[1] = 4.0
    expected[1, 2] = 7.0
    assert np.array_equal(T.data, expected)
    assert np.array_equal(S12.data, expected[1, 2])
    with pytest.raises(at.AcroError):
        at.SliceTensor(T, 3)
    with pytest.raises(at.AcroError):
        at.SliceTensor(T, 0, 0, 0)


def test_engine_moves_host_tensors_and_leaves_output_on_device(at, engine):
    A, B = at.Tensor(6), to_tensor(at, np.arange(6.0))
    engine("A_i = B_i", A, B)
    assert A.IsOnGPU() and B.IsOnGPU()
    A.MoveFromGPU()
    assert np.array_equal(A.data, np.arange(6.0))


def test_large_fill_and_scale(at):
    T = at.Tensor(1031, 257)
    T.SwitchToGPU()
    T.Set(1.5)
    T.Mult(-2.0)
    T.MoveFromGPU()
    assert np.all(T.data == -3.0)


@pytest.mark.parametrize("rows,cols", [(4, 1), (3, 7), (5, 8), (3, 1025)])
def test_fill_and_scale_of_slices_touch_exactly_their_entries(at, rows, cols):
    # slices start at any multiple of 8 bytes and have odd or even lengths; device fill and scale move 16 bytes per
    # lane and must neither miss the unaligned first / odd last entry nor touch a neighbour
    T = to_tensor(at, np.arange(rows * cols, dtype=np.float64).reshape(rows, cols))
    T.MoveToGPU()
    expected = T.data.copy()
    for r in range(rows):
        S = at.SliceTensor(T, r)
        if r % 2 == 0:
            S.Mult(-3.0)
            expected[r] *= -3.0
        else:
            S.Set(0.25 + r)
            expected[r] = 0.25 + r
    T.MoveFromGPU()
    assert np.array_equal(T.data, expected)


def test_page_locked_host_buffers_move_like_ordinary_ones(at):
    at.set_pinned_host_allocation(True)
    try:
        T = at.Tensor(257, 129)
    finally:
        at.set_pinned_host_allocation(False)
    U = at.Tensor(257, 129)                                     # ordinary again
    ref = np.arange(257 * 129, dtype=np.float64).reshape(257, 129)
    for X in (T, U):
        X.data[...] = ref
        X.MoveToGPU()
        X.Mult(2.0)
        X.MoveFromGPU()
        assert np.array_equal(X.data, 2.0 * ref)
    del T, U


def device_memory_in_use():
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return total.value - free.value


def test_device_mirror_of_a_tensor_over_a_callers_host_buffer_is_released(at):
    # the library allocated the mirror, so the library frees it, whoever owns the host buffer
    host = np.ones(8 << 20)                              # 64 MiB
    at.synchronize()
    before = device_memory_in_use()
    for _ in range(12):
        T = at.Tensor(host.size, hdata=host)
        T.MoveToGPU()
        T.Mult(2.0)
        T.MoveFromGPU()
        del T
    assert host[0] == 4096.0 and host[-1] == 4096.0
    assert device_memory_in_use() - before < 3 * host.nbytes


def test_callers_device_buffer_is_used_and_never_freed(at, engine):
    # a tensor over a caller's host AND device buffer, the device buffer at an odd offset (8-byte aligned only) of an
    # allocation that belongs to another tensor
    n = 1001
    pool = at.Tensor(4096)
    pool.data[...] = 0.0
    pool.MoveToGPU()
    base = pool.GetDeviceData()
    host = np.zeros(n)
    V = at.Tensor(n, hdata=host, ddata=base + 8 * 3, ongpu=True)
    assert V.IsMappedToGPU() and V.IsOnGPU() and V.GetDeviceData() == base + 24
    V.Set(2.0)
    X = to_tensor(at, np.arange(n, dtype=np.float64))
    engine("V_i += X_i", V, X)
    V.MoveFromGPU()
    assert np.array_equal(host, 2.0 + np.arange(n))
    V.UnmapFromGPU()                                     # lets go of the caller's buffer, does not free it
    assert not V.IsMappedToGPU()
    del V
    pool.MoveFromGPU()
    expected = np.zeros(4096)
    expected[3:3 + n] = 2.0 + np.arange(n)
    assert np.array_equal(pool.data, expected)
