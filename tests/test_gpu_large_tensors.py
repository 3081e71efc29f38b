"""Tensors with more than 2^31 entries (16 GiB of doubles): the reference indexes with int throughout
(tensor/Tensor.hpp:60, exec/CudaExecutor.cpp:437-474) and cannot hold them; a 288 GB device can.  Host buffers are
allocated but never touched here (values are set on the device), so the tests need device memory only."""
import numpy as np
import pytest

from acrotensor_amd import workloads
from gpu_helpers import rel_err

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


# ---- the schedules with kernels of their own, each with operands or results beyond 2^31 entries -----------------
# The big tensors are filled with ones on the device; a few entries (the first, those either side of entry 2^31 and the
# last) get small random integers through slices, so every expected value is exact and a 32-bit offset anywhere in a
# schedule's address arithmetic lands on the wrong entry.

COPY = {1: "S_i = P_i", 2: "S_i_j = P_i_j", 3: "S_i_j_k = P_i_j_k", 4: "S_i_j_k_l = P_i_j_k_l"}
SUM = {1: "S_i = A_e_i", 2: "S_i_j = A_e_i_j", 3: "S_i_j_k = A_e_i_j_k", 4: "S_i_j_k_l = A_e_i_j_k_l"}


def _ones(at, *dims):
    T = at.Tensor(*dims)
    T.SwitchToGPU()
    T.Set(1.0)
    return T


def _put(at, engine, T, e, values):
    P = at.Tensor(*values.shape)
    P.data[...] = values
    engine(COPY[values.ndim], at.SliceTensor(T, e), P)


def _take(at, engine, T, entries):
    shape = T.dims[1:]
    probe = at.Tensor(len(entries), *shape)
    probe.SwitchToGPU()
    for k, e in enumerate(entries):
        engine(COPY[len(shape)], at.SliceTensor(probe, k), at.SliceTensor(T, e))
    probe.MoveFromGPU()
    return probe.data.copy()


def _marked(E, per_entry):
    crossing = BEYOND // per_entry        # the entry that holds (or starts at) entry 2^31 of the tensor
    assert 1 < crossing < E - 2
    return [0, crossing - 1, crossing, crossing + 1, E - 1]


def _total(at, engine, A):
    S = at.Tensor(*A.dims[1:])
    engine(SUM[len(A.dims) - 1], S, A)
    S.MoveFromGPU()
    return S.data.copy()


@pytest.mark.parametrize("kernel,E,M,N,K,expect", [
    ("A_e_i_j = B_e_i_k C_e_k_j", 800000, 53, 53, 53, "product schedule on the FP64 matrix cores"),      # strips through LDS
    ("A_e_i_j = B_e_i_k C_e_j_k", 530000, 64, 64, 64, "product schedule on the FP64 matrix cores"),      # operands read directly
    ("A_e_i_j = B_e_i_k C_e_k_j", 132000, 128, 128, 128, "tiled product schedule"),
    ("A_e_i_j = B_e_i_k C_e_k_j", 34000000, 8, 8, 8, "operands staged in LDS"),
    ("A_e_i_j = B_e_i_k C_e_k_j", 135000000, 4, 4, 4, "operands staged in LDS"),
    ("A_e_i_j = B_e_i_k C_e_k_j", 600000, 61, 5, 61, "batch index e"),                                     # B alone beyond 2^31
])
def test_products_of_element_matrices_beyond_2_31_entries(at, kernel, E, M, N, K, expect):
    rng = np.random.default_rng(E)
    engine = at.TensorEngine("HIP")
    transposed = kernel.endswith("C_e_j_k")
    B, C, A = _ones(at, E, M, K), _ones(at, E, N, K) if transposed else _ones(at, E, K, N), at.Tensor(E, M, N)
    assert max(B.GetSize(), C.GetSize(), A.GetSize()) > BEYOND
    A.SwitchToGPU()
    A.Set(-1.0)
    marked = _marked(E, max(M * K, K * N, M * N))
    expected = {}
    for e in marked:
        bp, cp = rng.integers(-2, 3, (M, K)).astype(float), rng.integers(-2, 3, C.dims[1:]).astype(float)
        _put(at, engine, B, e, bp)
        _put(at, engine, C, e, cp)
        expected[e] = bp @ (cp.T if transposed else cp)
    engine(kernel, A, B, C)
    assert expect in engine.GetLastImplementation()
    got = _take(at, engine, A, marked + [1, E - 2])
    for k, e in enumerate(marked):
        assert np.array_equal(got[k], expected[e]), e
    assert np.all(got[-2:] == float(K))
    total = float(K) * (E - len(marked)) + sum(expected.values())
    assert np.array_equal(_total(at, engine, A), total)


@pytest.mark.parametrize("kernel,E,n,comps", [
    ("A_e_i = B_i_j X_e_j", 34000000, 64, 0),           # results stored from the accumulators
    ("A_e_i = B_i_j X_e_j", 110000000, 20, 0),          # padded operator, results written out through LDS
    ("A_e_i_k = B_i_j X_e_j_k", 12000000, 64, 3),       # three components per vector element
])
def test_operator_on_the_matrix_cores_beyond_2_31_entries(at, kernel, E, n, comps):
    rng = np.random.default_rng(n + comps)
    engine = at.TensorEngine("HIP")
    shape = (n, comps) if comps else (n,)
    X, A, B = _ones(at, E, *shape), at.Tensor(E, *shape), at.Tensor(n, n)
    assert X.GetSize() > BEYOND
    A.SwitchToGPU()
    A.Set(-1.0)
    B.data[...] = rng.integers(-3, 4, (n, n))
    marked = _marked(E, X.GetSize() // E)
    expected = {}
    for e in marked:
        xp = rng.integers(-2, 3, shape).astype(float)
        _put(at, engine, X, e, xp)
        expected[e] = B.data @ xp
    engine(kernel, A, B, X)
    assert "operator schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    got = _take(at, engine, A, marked + [1, E - 2])
    plain = B.data @ np.ones(shape)
    for k, e in enumerate(marked):
        assert np.array_equal(got[k], expected[e]), e
    assert np.array_equal(got[-2], plain) and np.array_equal(got[-1], plain)
    assert np.array_equal(_total(at, engine, A), plain * (E - len(marked)) + sum(expected.values()))


def test_gram_matrix_and_matrix_times_vector_beyond_2_31_entries(at):
    rng = np.random.default_rng(5)
    engine = at.TensorEngine("HIP")
    E, n = 34000000, 64
    B, C, G = _ones(at, E, n), _ones(at, E, n), at.Tensor(n, n)
    marked = _marked(E, n)
    expected = np.full((n, n), float(E - len(marked)))
    for e in marked:
        bp, cp = rng.integers(-2, 3, n).astype(float), rng.integers(-2, 3, n).astype(float)
        _put(at, engine, B, e, bp)
        _put(at, engine, C, e, cp)
        expected += np.outer(bp, cp)
    engine("G_i_j = B_e_i C_e_j", G, B, C)
    assert "Gram schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    G.MoveFromGPU()
    assert np.array_equal(G.data, expected)
    del B, C
    # an element matrix of odd size times an element vector: the product schedule with a single column
    E, n = 3000000, 27
    M, X, Y = _ones(at, E, n, n), _ones(at, E, n), at.Tensor(E, n)
    assert M.GetSize() > BEYOND
    marked = _marked(E, n * n)
    products = {}
    for e in marked:
        mp, xp = rng.integers(-2, 3, (n, n)).astype(float), rng.integers(-2, 3, n).astype(float)
        _put(at, engine, M, e, mp)
        _put(at, engine, X, e, xp)
        products[e] = mp @ xp
    engine("Y_e_i = M_e_i_j X_e_j", Y, M, X)
    assert "product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    Y.MoveFromGPU()
    want = np.full((E, n), float(n))
    for e in marked:
        want[e] = products[e]
    assert np.array_equal(Y.data, want)


def test_transposes_beyond_2_31_entries(at):
    rng = np.random.default_rng(6)
    engine = at.TensorEngine("HIP")
    n = 47000                                            # 2.2e9 entries
    B, A = at.Tensor(n, n), at.Tensor(n, n)
    for T in (A, B):
        T.SwitchToGPU()
    B.Set(0.0)
    A.Set(-1.0)
    rows = [0, BEYOND // n, BEYOND // n + 1, n - 1]      # rows of B: columns of A
    values = {j: rng.integers(1, 9, n).astype(float) for j in rows}
    for j in rows:
        _put(at, engine, B, j, values[j])
    engine("A_i_j = B_j_i", A, B)
    assert "transpose schedule" in engine.GetLastImplementation()
    picked = [0, 1, BEYOND // n, BEYOND // n + 1, n - 2, n - 1]
    got = _take(at, engine, A, picked)
    for k, i in enumerate(picked):
        want = np.zeros(n)
        for j in rows:
            want[j] = values[j][i]
        assert np.array_equal(got[k], want), i
    S = at.Tensor(n)
    engine("S_j = A_i_j", S, A)                          # column sums of A: row sums of B
    S.MoveFromGPU()
    want = np.zeros(n)
    for j in rows:
        want[j] = values[j].sum()
    assert np.array_equal(S.data, want)
    del A, B
    # per entry: 32 x 32 matrices
    E, m = 2200000, 32
    B, A = _ones(at, E, m, m), at.Tensor(E, m, m)
    A.SwitchToGPU()
    A.Set(-1.0)
    marked = _marked(E, m * m)
    patterns = {e: rng.integers(-4, 5, (m, m)).astype(float) for e in marked}
    for e in marked:
        _put(at, engine, B, e, patterns[e])
    engine("A_e_i_j = B_e_j_i", A, B)
    assert "transpose schedule" in engine.GetLastImplementation()
    got = _take(at, engine, A, marked + [E - 2])
    for k, e in enumerate(marked):
        assert np.array_equal(got[k], patterns[e].T), e
    assert np.all(got[-1] == 1.0)
    assert np.array_equal(_total(at, engine, A), float(E - len(marked)) + sum(p.T for p in patterns.values()))


def test_fused_mass_apply_beyond_2_31_entries(at, checker):
    # the sum-factorised mass apply (seven kernels in one launch, intermediates in LDS) over 17.5 million elements: the
    # geometric factors are 2.18e9 entries.  The inputs are 34 100 copies of a 512-element workload, laid out on the
    # device, so every copy of the result must equal the first bit for bit and the first must match the checker.
    engine = at.TensorEngine("HIP")
    wl, times = workloads.config4(E=512), 34100
    tensors = workloads.bind_to_engine_repeated(wl, at, engine, times)
    assert tensors["D"].GetSize() > BEYOND
    tensors["Y"].Set(-1.0)
    workloads.launch(wl, engine, tensors)
    Y = tensors["Y"]
    per_copy = Y.GetSize() // times
    Y.Reshape(times, per_copy)
    crossing = BEYOND // (512 * 125)                     # the copy whose geometric factors hold entry 2^31
    picked = [0, 1, crossing - 1, crossing, crossing + 1, times - 1]
    got = _take(at, engine, Y, picked)
    expected = workloads.run_on_checker(wl, checker)["Y"].reshape(-1)
    assert rel_err(got[0], expected) <= 1e-12
    for k in range(1, len(picked)):
        assert np.array_equal(got[k], got[0]), picked[k]
    assert rel_err(_total(at, engine, Y), times * expected) <= 1e-12


def test_batched_inverse_and_determinant_beyond_2_31_entries(at, checker):
    engine = at.TensorEngine("HIP")
    small, times = workloads.config2_inputs(E=250, Q=4), 240000          # 1 000 Jacobians, 240 000 times: 2.16e9 entries
    S = at.Tensor(*small.shape)
    S.data[...] = small
    J = at.Tensor(times, *small.shape)
    J.SwitchToGPU()
    engine("R_t_e_q_i_j = S_e_q_i_j", J, S)
    assert J.GetSize() > BEYOND
    J.Reshape(times * 1000, 3, 3)
    Jinv, Jdet = at.Tensor(times * 1000, 3, 3), at.Tensor(times * 1000)
    for T in (Jinv, Jdet):
        T.SwitchToGPU()
        T.Set(-1.0)
    engine.BatchMatrixInvDet(Jinv, Jdet, J)
    Jinv.Reshape(times, 1000, 3, 3)
    Jdet.Reshape(times, 1000)
    crossing = BEYOND // 9000
    picked = [0, crossing - 1, crossing, crossing + 1, times - 1]
    ri, rd = checker.batch_matrix_inv_det(small)
    inv, det = _take(at, engine, Jinv, picked), _take(at, engine, Jdet, picked)
    for k in range(len(picked)):
        assert np.array_equal(inv[k], ri.reshape(1000, 3, 3)) and np.array_equal(det[k], rd.reshape(1000)), picked[k]
    assert rel_err(_total(at, engine, Jinv), times * ri.reshape(1000, 3, 3)) <= 1e-12
