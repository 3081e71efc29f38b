"""Batched matrix inverses and determinants recorded inside a multi-kernel launch: they become kernels of the fused
launch when a later kernel reads their result (the geometric-factor setup of the reference's
unittest/kernel/test_TensorEngine.cpp:498-590 is then one launch from the Jacobians to D).  Expected values: the
checker's batched inverse / determinant (bit for bit, as for the operations run on their own) followed by the
checker's contraction (1e-12 relative to the largest entry)."""
import numpy as np
import pytest

from gpu_helpers import rel_err, to_tensor

pytestmark = pytest.mark.gpu
TOL = 1e-12

GEOMETRIC_FACTORS = {
    3: "D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j",
    2: "D_e_m_n_k1_k2 = W_k1_k2 C_e_k1_k2 Jdet_e_k1_k2 Jinv_e_k1_k2_n_j Jinv_e_k1_k2_m_j",
    1: "D_e_m_n_k1 = W_k1 C_e_k1 Jdet_e_k1 Jinv_e_k1_n_j Jinv_e_k1_m_j",
}


def jacobians(rng, E, Q, dim):
    pts = (Q,) * dim
    J = np.eye(dim) + 0.2 * rng.uniform(-1, 1, (E,) + pts + (dim, dim))
    return J, rng.uniform(0.1, 1.0, pts), rng.uniform(0.5, 1.5, (E,) + pts)


def expected_factors(checker, dim, J, W, C):
    ji, jd = checker.batch_matrix_inv_det(J)
    D = np.zeros((J.shape[0], dim, dim) + J.shape[1:1 + dim])
    checker.contract(GEOMETRIC_FACTORS[dim], D, W, C, jd, ji, ji)
    return ji, jd, D


@pytest.mark.parametrize("transient", [True, False])
@pytest.mark.parametrize("E,Q,dim", [(7, 4, 3), (1, 10, 3), (37, 3, 2), (5, 6, 1), (300, 1, 3)])
def test_geometric_factors_in_one_launch(at, engine, checker, E, Q, dim, transient):
    print("case:", E, Q, dim, transient, flush=True)
    J, W, C = jacobians(np.random.default_rng(100 * E + 10 * Q + dim), E, Q, dim)
    pts = (Q,) * dim
    tJ, tW, tC = to_tensor(at, J), to_tensor(at, W), to_tensor(at, C)
    Jinv, Jdet, D = at.Tensor(E, *pts, dim, dim), at.Tensor(E, *pts), at.Tensor(E, dim, dim, *pts)
    for t in (Jinv, Jdet, D):
        t.data[...] = -7.0
        t.MoveToGPU()
    Jinv.SetTransient(transient)
    Jdet.SetTransient(transient)
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
    engine(GEOMETRIC_FACTORS[dim], D, tW, tC, Jdet, Jinv, Jinv)
    engine.EndMultiKernelLaunch()
    src = engine.GetLastImplementation()
    assert src.count("__global__") == 1 and "Jinv<-registers" in src and "Jdet<-registers" in src
    D.MoveFromGPU()
    ji, jd, expected = expected_factors(checker, dim, J, W, C)
    assert rel_err(D.data, expected) <= TOL
    if not transient:
        Jinv.MoveFromGPU()
        Jdet.MoveFromGPU()
        assert np.array_equal(Jinv.data, ji) and np.array_equal(Jdet.data, jd)      # bit for bit


@pytest.mark.parametrize("m", [1, 2, 3])
def test_inverse_alone_and_determinant_alone_with_a_reader(at, engine, checker, m):
    rng = np.random.default_rng(m)
    A = np.eye(m) + 0.2 * rng.uniform(-1, 1, (41, 6, m, m))
    V = rng.uniform(-1, 1, (41, 6, m))
    ri, rd = checker.batch_matrix_inv_det(A)
    tA, tV = to_tensor(at, A), to_tensor(at, V)
    # X = Ainv V, the inverse recorded alone
    Ainv, X = at.Tensor(41, 6, m, m), at.Tensor(41, 6, m)
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixInverse(Ainv, tA)
    engine("X_e_k_i = Ainv_e_k_i_j V_e_k_j", X, Ainv, tV)
    engine.EndMultiKernelLaunch()
    assert "(matrix inverse)" in engine.GetLastImplementation() and "Ainv<-registers" in engine.GetLastImplementation()
    X.MoveFromGPU()
    Ainv.MoveFromGPU()
    assert np.array_equal(Ainv.data, ri)
    expected = np.zeros((41, 6, m))
    checker.contract("X_e_k_i = Ainv_e_k_i_j V_e_k_j", expected, ri, V)
    assert rel_err(X.data, expected) <= TOL
    # S = det(A) V, the determinant recorded alone
    Adet, S = at.Tensor(41, 6), at.Tensor(41, 6, m)
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixDet(Adet, tA)
    engine("S_e_k_i = Adet_e_k V_e_k_i", S, Adet, tV)
    engine.EndMultiKernelLaunch()
    assert "(determinant)" in engine.GetLastImplementation()
    S.MoveFromGPU()
    Adet.MoveFromGPU()
    assert np.array_equal(Adet.data, rd)
    assert rel_err(S.data, rd[..., None] * V) <= TOL


def test_reader_that_is_not_the_next_kernel_and_reader_with_other_index_names(at, engine, checker):
    rng = np.random.default_rng(5)
    E, K = 9, 5
    A = np.eye(3) + 0.2 * rng.uniform(-1, 1, (E, K, 3, 3))
    V, B = rng.uniform(-1, 1, (E, K, 3)), rng.uniform(-1, 1, (E, 4))
    ri, rd = checker.batch_matrix_inv_det(A)
    tA, tV, tB = to_tensor(at, A), to_tensor(at, V), to_tensor(at, B)
    Ainv, Adet, X, Y, Z = at.Tensor(E, K, 3, 3), at.Tensor(E, K), at.Tensor(E, K, 3), at.Tensor(E, 4), at.Tensor(E, K)
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixInvDet(Ainv, Adet, tA)
    engine("Y_e_i = B_e_i B_e_i", Y, tB, tB)                     # unrelated kernel in between
    engine("X_e_k_i = Ainv_e_k_j_i V_e_k_j", X, Ainv, tV)        # transposed use of the inverse
    engine("Z_e_q = Adet_e_q Adet_e_q", Z, Adet, Adet)           # the determinant under another index name
    engine.EndMultiKernelLaunch()
    for t in (Ainv, Adet, X, Y, Z):
        t.MoveFromGPU()
    assert np.array_equal(Ainv.data, ri) and np.array_equal(Adet.data, rd)
    assert rel_err(X.data, np.einsum("ekji,ekj->eki", ri, V)) <= TOL
    assert rel_err(Y.data, B * B) <= TOL and rel_err(Z.data, rd * rd) <= TOL


def test_operation_without_reader_in_the_launch_and_in_place_inverse(at, engine, checker):
    rng = np.random.default_rng(6)
    A = np.eye(3) + 0.2 * rng.uniform(-1, 1, (50, 3, 3))
    V = rng.uniform(-1, 1, (50, 3))
    ri, rd = checker.batch_matrix_inv_det(A)
    tA, tV = to_tensor(at, A), to_tensor(at, V)
    Ainv, Adet, X = at.Tensor(50, 3, 3), at.Tensor(50), at.Tensor(50, 3)
    engine.BeginMultiKernelLaunch()
    engine("X_e_i = V_e_i V_e_i", X, tV, tV)
    engine.BatchMatrixInvDet(Ainv, Adet, tA)                      # nobody reads it: runs on its own, after the kernel
    engine.EndMultiKernelLaunch()
    for t in (Ainv, Adet, X):
        t.MoveFromGPU()
    assert np.array_equal(Ainv.data, ri) and np.array_equal(Adet.data, rd) and rel_err(X.data, V * V) <= TOL
    # in place: the operand is overwritten by its inverse, then read
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixInverse(tA, tA)
    engine("X_e_i = A_e_i_j V_e_j", X, tA, tV)
    engine.EndMultiKernelLaunch()
    X.MoveFromGPU()
    tA.MoveFromGPU()
    assert np.array_equal(tA.data, ri)
    assert rel_err(X.data, np.einsum("eij,ej->ei", ri, V)) <= TOL


def test_single_matrix_without_leading_dimensions(at, engine, checker):
    A = np.array([[2.0, 1.0, 0.5], [0.25, 3.0, 1.0], [1.0, 0.5, 4.0]])
    ri, _ = checker.batch_matrix_inv_det(A.reshape(1, 3, 3))
    tA, Ainv, I = to_tensor(at, A), at.Tensor(3, 3), at.Tensor(3, 3)
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixInverse(Ainv, tA)
    engine("I_i_k = Ainv_j_i A_j_k", I, Ainv, tA)                 # the reference's layout: A^T-inverse for 3 x 3
    engine.EndMultiKernelLaunch()
    I.MoveFromGPU()
    Ainv.MoveFromGPU()
    assert np.array_equal(Ainv.data, ri.reshape(3, 3))
    assert np.abs(I.data - np.eye(3)).max() < 1e-13


def test_recorded_matrix_operations_replay_from_a_recorded_launch_sequence(at, engine, checker):
    E, Q = 11, 4
    J, W, C = jacobians(np.random.default_rng(8), E, Q, 3)
    tJ, tW, tC = to_tensor(at, J), to_tensor(at, W), to_tensor(at, C)
    Jinv, Jdet, D = at.Tensor(E, Q, Q, Q, 3, 3), at.Tensor(E, Q, Q, Q), at.Tensor(E, 3, 3, Q, Q, Q)
    Jinv.SetTransient(True)
    Jdet.SetTransient(True)

    def step():
        engine.BeginMultiKernelLaunch()
        engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
        engine(GEOMETRIC_FACTORS[3], D, tW, tC, Jdet, Jinv, Jinv)
        engine.EndMultiKernelLaunch()

    step()
    _, _, expected = expected_factors(checker, 3, J, W, C)
    with at.recorded_launches() as recording:
        step()
    for _ in range(3):
        D.MoveToGPU()
        D.Set(0.0)                                                # eager work between the replays
        recording.launch()
        D.MoveFromGPU()
        assert rel_err(D.data, expected) <= TOL


def test_geometric_factors_at_full_size(at, engine, checker):
    # E = 16384 elements of 10^3 points (the size bench.py measures): a sample of elements against the checker, and
    # on every point the symmetry of D and its closed form where the Jacobian is diagonal
    E, Q = 16384, 10
    rng = np.random.default_rng(77)
    J = rng.uniform(-0.2, 0.2, (E, Q, Q, Q, 3, 3))
    J[..., 0, 0] += 1.0
    J[..., 1, 1] += 1.5
    J[..., 2, 2] += 2.0
    diagonal = np.arange(0, E, 97)                  # these elements get diagonal Jacobians
    for a in range(3):
        for b in range(3):
            if a != b:
                J[diagonal, ..., a, b] = 0.0
    W, C = rng.uniform(0.1, 1.0, (Q, Q, Q)), rng.uniform(0.5, 1.5, (E, Q, Q, Q))
    tJ, tW, tC = to_tensor(at, J), to_tensor(at, W), to_tensor(at, C)
    Jinv, Jdet, D = at.Tensor(E, Q, Q, Q, 3, 3), at.Tensor(E, Q, Q, Q), at.Tensor(E, 3, 3, Q, Q, Q)
    Jinv.SetTransient(True)
    Jdet.SetTransient(True)
    print("launch", flush=True)
    engine.BeginMultiKernelLaunch()
    engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
    engine(GEOMETRIC_FACTORS[3], D, tW, tC, Jdet, Jinv, Jinv)
    engine.EndMultiKernelLaunch()
    D.MoveFromGPU()
    got = D.data
    assert np.array_equal(got, got.transpose(0, 2, 1, 3, 4, 5))          # D_mn = D_nm, bit for bit
    sample = np.unique(np.concatenate([[0, 1, E // 2, E - 1], rng.integers(0, E, 12)]))
    _, _, expected = expected_factors(checker, 3, np.ascontiguousarray(J[sample]), W, np.ascontiguousarray(C[sample]))
    assert rel_err(got[sample], expected) <= TOL
    d = np.stack([J[diagonal, ..., a, a] for a in range(3)], axis=1)     # [elements, 3, Q, Q, Q]
    closed = (W * C[diagonal] * d[:, 0] * d[:, 1] * d[:, 2])[:, None] / d ** 2
    for a in range(3):
        assert rel_err(got[diagonal, a, a], closed[:, a]) <= TOL
        for b in range(3):
            if a != b:
                assert not got[diagonal, a, b].any()
