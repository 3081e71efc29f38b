"""The plain-C restatement against the reference itself (oracle/_ref, compiled from the reference's sources):
bit-for-bit on seeded random inputs, including the reference's quirks."""
import numpy as np
import pytest

from acrotensor_amd import workloads

KERNELS = [
    ("A_i = B_i", [(9,)]),
    ("A_i = B_i_i", [(6, 6)]),
    ("A_i = B_j_j", [(5, 5)]),
    ("A_i = C_i_j B_j", [(13, 17), (17,)]),
    ("A_i_j = B_j_i", [(8, 5)]),
    ("A_i_j = B_i_k B_j_k", [(6, 4), (6, 4)]),
    ("S_i_j = A_n_i_j B_n", [(4096, 3, 3), (4096,)]),
    ("A_e_i += B_e_i_j_k C_j D_k", [(5, 4, 3, 6), (3,), (6,)]),
    ("A_e_i -= B_e_i_j_k C_j D_k", [(5, 4, 3, 6), (3,), (6,)]),
    ("S_e_i1_i2_j1_j2 = B_i1_j1_k1_m_n B_i2_j2_k2_m_n D_e_k1_k2_m_n",
     [(3, 3, 4, 2, 2), (3, 3, 4, 2, 2), (5, 4, 4, 2, 2)]),
    ("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s", [(4, 3)] * 6 + [(5, 4, 4, 4)]),
]


def shape_of_output(kernel, shapes):
    lhs, rhs = kernel.replace("+=", "=").replace("-=", "=").split("=")
    sizes = {}
    for var, shp in zip(rhs.split(), shapes):
        for name, n in zip(var.split("_")[1:], shp):
            sizes[name] = n
    return tuple(sizes.get(n, 3) for n in lhs.split()[0].split("_")[1:])


@pytest.mark.parametrize("kernel,shapes", KERNELS)
def test_contraction_bit_for_bit(checker, reference, kernel, shapes):
    rng = np.random.default_rng(abs(hash(kernel)) % 2 ** 31)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    init = rng.uniform(-1, 1, shape_of_output(kernel, shapes))
    a, b = init.copy(), init.copy()
    checker.contract(kernel, a, *ins)
    reference.contract(kernel, b, *ins)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("make", [lambda: workloads.config1(n=2048), lambda: workloads.config3(E=4),
                                  lambda: workloads.config4(E=8), lambda: workloads.config5(E=2, Q=5, P=4)])
def test_configs_bit_for_bit(checker, reference, make):
    wl = make()
    a = workloads.run_on_checker(wl, checker)
    b = workloads.run_on_checker(wl, reference)
    for name in a:
        assert np.array_equal(a[name], b[name]), name


def test_rejections_agree(checker, reference):
    for c in (checker, reference):
        with pytest.raises(RuntimeError):
            c.contract("A_i=B_iC_i", np.zeros(3), np.zeros(3), np.zeros(2))
        with pytest.raises(RuntimeError):
            c.contract("B_lah=A_lah_", np.zeros(3), np.zeros(3))


@pytest.mark.parametrize("m", [1, 2, 3])
def test_small_matrix_ops_bit_for_bit(checker, reference, m):
    rng = np.random.default_rng(10 + m)
    A = np.eye(m) + 0.1 * rng.uniform(-1, 1, (64, 5, m, m))      # non-symmetric on purpose
    for op in ("batch_matrix_inverse", "batch_matrix_det"):
        assert np.array_equal(getattr(checker, op)(A), getattr(reference, op)(A))
    a, b = checker.batch_matrix_inv_det(A), reference.batch_matrix_inv_det(A)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_three_by_three_inverse_is_the_transposed_inverse_in_the_reference(reference):
    rng = np.random.default_rng(3)
    A = np.eye(3) + 0.2 * rng.uniform(-1, 1, (8, 3, 3))
    R = reference.batch_matrix_inverse(A)
    assert np.allclose(np.einsum("nij,nkj->nik", A, R), np.eye(3), atol=1e-13)      # A R^T = I
    assert not np.allclose(np.einsum("nij,njk->nik", A, R), np.eye(3), atol=1e-3)   # A R != I


def test_scatter_gather_and_inverse_map_bit_for_bit(checker, reference):
    rng = np.random.default_rng(21)
    domain, rng_size = 40, 100
    M = np.concatenate([np.arange(domain), rng.integers(0, domain, rng_size - domain)]).astype(np.int32)
    rng.shuffle(M)                                               # every domain entry keeps a preimage
    src, vals = rng.uniform(-1, 1, domain), rng.uniform(-1, 1, rng_size)
    assert np.array_equal(checker.scatter(src, M), reference.scatter(src, M))
    assert np.array_equal(checker.sum_gather(vals, M, domain), reference.sum_gather(vals, M, domain))
    a, b = checker.index_mapping_inverse(M, domain), reference.index_mapping_inverse(M, domain)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    # also for a map that leaves domain entries without preimage (the reference's offset walk is restated as is)
    M2 = (M % 7 * 3).astype(np.int32)
    a, b = checker.index_mapping_inverse(M2, domain), reference.index_mapping_inverse(M2, domain)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
