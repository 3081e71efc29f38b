"""Tensors with more than 2^31 entries (16 GiB of doubles): the reference indexes with int throughout
(tensor/Tensor.hpp:60, exec/CudaExecutor.cpp:437-474) and cannot hold them; a 288 GB device can.  Host buffers are
allocated but never touched here (values are set on the device), so the tests need device memory only."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

BEYOND = 1 << 31


def test_fill_scale_and_slices_beyond_2_31_entries(at):
    E, I = 33000, 65600                      # 2.16e9 entries, 17.3 GB
    T = at.Tensor(E, I)
    assert T.GetSize() == E * I > BEYOND and T.GetStride(0) == I
    T.SwitchToGPU()
    T.Set(1.5)
    T.Mult(2.0)
    last, first = at.SliceTensor(T, E - 1), at.SliceTensor(T, 0)
    last.Set(-7.0)                           # starts 2.16e9 entries into the tensor
    probe = at.Tensor(3, I)
    probe.SwitchToGPU()
    engine = at.TensorEngine("HIP")
    engine("P_i = S_i", at.SliceTensor(probe, 0), first)
    engine("P_i = S_i", at.SliceTensor(probe, 1), at.SliceTensor(T, E - 2))
    engine("P_i = S_i", at.SliceTensor(probe, 2), last)
    probe.MoveFromGPU()
    assert np.all(probe.data[0] == 3.0) and np.all(probe.data[1] == 3.0) and np.all(probe.data[2] == -7.0)


def test_contraction_over_a_tensor_beyond_2_31_entries(at):
    # unrolled path: element offsets e * 65536 + i * 8 pass 2^31 for e >= 32768
    E, I, J = 33000, 8192, 8
    B, V, C = at.Tensor(E, I, J), at.Tensor(J), at.Tensor(E, I)
    assert B.GetSize() > BEYOND
    B.SwitchToGPU()
    B.Set(1.0)
    for e, value in ((32767, 2.0), (32768, 3.0), (E - 1, 4.0)):
        at.SliceTensor(B, e).Set(value)
    V.data[...] = np.arange(1.0, J + 1)
    engine = at.TensorEngine("HIP")
    engine("C_e_i = B_e_i_j V_j", C, B, V)
    assert "const long o_k0v0" in engine.GetLastImplementation()
    C.MoveFromGPU()
    expected = np.full(E, 36.0)
    expected[32767], expected[32768], expected[E - 1] = 72.0, 108.0, 144.0
    assert np.array_equal(C.data, np.repeat(expected[:, None], I, axis=1))


def test_split_contraction_and_counted_loops_beyond_2_31_entries(at):
    engine = at.TensorEngine("HIP")
    # reduction schedule: S_i = sum over n of A_n_i W_n with 2.4e9 entries of A
    n = (1 << 28) + 5
    A, W, S = at.Tensor(n, 9), at.Tensor(n), at.Tensor(9)
    for t, v in ((A, 0.5), (W, 2.0)):
        t.SwitchToGPU()
        t.Set(v)
    at.SliceTensor(A, n - 1).Set(100.5)      # the very last row, 2.4e9 entries in
    engine("S_i = A_n_i W_n", S, A, W)
    S.MoveFromGPU()
    assert np.array_equal(S.data, np.full(9, float(n - 1) + 201.0))
    del A, W
    # counted loops: 70 000 terms per output, 2.3e9 entries
    E, J = 33000, 70000
    B, V, C = at.Tensor(E, J), at.Tensor(J), at.Tensor(E)
    B.SwitchToGPU()
    B.Set(0.25)
    at.SliceTensor(B, E - 1).Set(0.5)
    V.Set(4.0)
    engine("C_e = B_e_j V_j", C, B, V)
    assert "looped" in engine.GetLastImplementation()
    C.MoveFromGPU()
    expected = np.full(E, float(J))
    expected[E - 1] = 2.0 * J
    assert np.array_equal(C.data, expected)
