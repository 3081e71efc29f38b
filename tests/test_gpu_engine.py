"""The reference's engine suite (unittest/kernel/test_TensorEngine.cpp) re-expressed for the "HIP" policy, driven
through the C ABI.  Expected values come from the checker (the restated CPU interpreter) and, as in the reference's
tests, from closed forms.  Integer-valued inputs make results exact in fp64 whatever the summation order, so those
comparisons are bit-exact (index mapping); random inputs are held to 1e-12 relative to the largest entry."""
import numpy as np
import pytest

from gpu_helpers import output_shape, rel_err, run_single, to_tensor

pytestmark = pytest.mark.gpu
TOL = 1e-12


def seq(shape, mod=None, scale=1.0):
    a = np.arange(int(np.prod(shape)), dtype=np.float64)
    if mod:
        a = a % mod
    return (a * scale).reshape(shape)


def test_assert_compatible_dimensions(at, engine):
    # unittest/kernel/test_TensorEngine.cpp:37-47
    T1out_3, T1_3, T1_2, T2_3_3 = at.Tensor(3), at.Tensor(3), at.Tensor(2), at.Tensor(3, 3)
    for t in (T1_3, T1_2, T2_3_3):
        t.Set(1.0)
    engine("A_i=B_iC_i", T1out_3, T1_3, T1_3)
    with pytest.raises(at.AcroError):
        engine("A_i=B_iC_i", T1out_3, T1_3, T1_2)
    engine("A_i=B_i_jC_i", T1out_3, T2_3_3, T1_3)
    with pytest.raises(at.AcroError):
        engine("A_i=B_i_jC_i", T1out_3, T2_3_3, T1_2)
    with pytest.raises(at.AcroError):
        engine("A_i=B_i_jC_i", T1out_3, T2_3_3)                 # wrong number of inputs
    with pytest.raises(at.AcroError):
        engine("A_i_j=B_i_jC_i", T1out_3, T2_3_3, T1_3)         # wrong output rank
    with pytest.raises(at.AcroError):
        engine("Blah=Alah", T1out_3, T1_3)
    with pytest.raises(at.AcroError):
        engine.EndMultiKernelLaunch()                           # End without Begin
    engine.BeginMultiKernelLaunch()
    with pytest.raises(at.AcroError):
        engine.BeginMultiKernelLaunch()                         # Begin twice
    engine.EndMultiKernelLaunch()                               # empty capture is a no-op


BASIC = [
    ("A_i=B_i", [(3,)]),                       # simple copy
    ("A_i=B_i_i", [(3, 3)]),                   # diagonal
    ("A_i=B_j_j", [(3, 3)]),                   # contraction + broadcast
    ("A_i = C_i_j B_j", [(3, 3), (3,)]),       # matvec
    ("A_i_j=B_j_i", [(4, 4)]),                 # transpose
    ("A_m_n=B_m_j B_n_j", [(3, 3), (3, 3)]),   # B B^T (same tensor under one name, see below)
    ("A_i=B_j_k_l_m_n", [(1, 2, 1, 3, 2)]),    # singleton dimensions, everything contracted
    ("A_i_j_k = B_k_j_i", [(5, 1, 7)]),
    ("A_e_i = B_e_i_j_k C_j D_k", [(17, 4, 5, 2), (5,), (2,)]),
    ("A_i_j = B_i_k C_k_j", [(33, 65), (65, 17)]),
    ("A_i_i = B_i", [(4,)]),                   # repeated output index: only the diagonal is written
]


@pytest.mark.parametrize("kernel,shapes", BASIC)
def test_basic_computations_exact_on_integer_data(at, engine, checker, kernel, shapes):
    ins = [seq(s, mod=11) - 3.0 for s in shapes]
    if kernel.startswith("A_m_n"):
        ins[1] = ins[0]
    init = np.full(output_shape(kernel, shapes), 7.0)
    got, expected = run_single(at, engine, checker, kernel, init, *ins)
    assert np.array_equal(got, expected)


def test_same_name_bound_to_one_tensor(at, engine):
    B = to_tensor(at, seq((3, 3)))
    A = at.Tensor(3, 3)
    engine("A_m_n=B_m_j B_n_j", A, B, B)
    A.MoveFromGPU()
    assert np.array_equal(A.data, B.data @ B.data.T)


@pytest.mark.parametrize("kernel,shapes", BASIC[:6] + [("A_i += B_i_j C_j", [(300, 7), (7,)]),
                                                       ("A_e_i += B_e_i_j_k C_j D_k", [(17, 4, 5, 2), (5,), (2,)])])
def test_basic_computations_random_data(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(abs(hash(kernel)) % 2 ** 31)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    init = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, init, *ins)
    assert rel_err(got, expected) <= TOL


def test_minus_equal_subtracts(at, engine, checker):
    # The reference's device generator honours "-=" (exec/CudaExecutor.cpp:534-536) while its host interpreter adds
    # (exec/CPUInterpretedExecutor.cpp:106); the HIP policy subtracts, i.e. init - (what "+=" would add).
    rng = np.random.default_rng(11)
    B, C, init = rng.uniform(-1, 1, (40, 6)), rng.uniform(-1, 1, 6), rng.uniform(-1, 1, 40)
    got, added = run_single(at, engine, checker, "A_i -= B_i_j C_j", init, B, C)
    assert rel_err(got, init - (added - init)) <= TOL


def test_multi_kernel_launch_second_kernel_overwrites_first(at, engine):
    # unittest/kernel/test_TensorEngine.cpp:211-228
    A, B1, B2, C = at.Tensor(3), at.Tensor(3), at.Tensor(3), at.Tensor(3, 3)
    B1.data[...] = [1.0, 2.0, 3.0]
    B2.Set(1.0)
    C.Set(1.0)
    engine.BeginMultiKernelLaunch()
    engine("A_i = B1_i", A, B1)
    engine("A_i = C_i_j B2_j", A, C, B2)
    engine.EndMultiKernelLaunch()
    A.MoveFromGPU()
    assert np.array_equal(A.data, [3.0, 3.0, 3.0])


def test_multi_kernel_launch_without_common_outer_index_runs_kernel_by_kernel(at, engine):
    A, B, C, D = at.Tensor(4), to_tensor(at, seq((4,))), at.Tensor(6), to_tensor(at, seq((6,)))
    engine.BeginMultiKernelLaunch()
    engine("A_i = B_i", A, B)
    engine("C_j = D_j", C, D)
    engine.EndMultiKernelLaunch()
    assert "not fused" in engine.GetLastImplementation()
    A.MoveFromGPU()
    C.MoveFromGPU()
    assert np.array_equal(A.data, B.data) and np.array_equal(C.data, D.data)


def test_2d_mass_matrix(at, engine, checker):
    # unittest/kernel/test_TensorEngine.cpp:232-309
    rng = np.random.default_rng(2)
    B, W, T = seq((3, 2)), seq((3, 3)) + 1.0, rng.uniform(0.5, 1.5, (5, 3, 3))
    D, expD = run_single(at, engine, checker, "D_e_k1_k2 = W_k1_k2 T_e_k1_k2", np.zeros((5, 3, 3)), W, T)
    assert rel_err(D, W[None] * T) <= TOL
    M, expM = run_single(at, engine, checker, "M_e_i1_i2_j1_j2=B_k1_i1 B_k1_j1 B_k2_i2 B_k2_j2 D_e_k1_k2",
                         np.zeros((5, 2, 2, 2, 2)), B, B, B, B, D)
    assert rel_err(M, expM) <= TOL
    assert rel_err(M, np.einsum("ai,aj,bk,bl,eab->eikjl", B, B, B, B, D)) <= TOL


def test_2d_stiffness_partial_assembly_with_slices(at, engine, checker):
    # unittest/kernel/test_TensorEngine.cpp:311-435: integer-valued data, slices as outputs and inputs
    B, G, X, D = seq((4, 4)), seq((4, 4), scale=0.5), seq((5, 4, 4)), seq((5, 2, 2, 4, 4))
    tB, tG, tX, tD = (to_tensor(at, a) for a in (B, G, X, D))
    T, U, Z, Y = at.Tensor(5, 4, 4), at.Tensor(2, 5, 4, 4), at.Tensor(2, 5, 4, 4), at.Tensor(5, 4, 4)
    U1, U2 = at.SliceTensor(U, 0), at.SliceTensor(U, 1)
    Z1, Z2 = at.SliceTensor(Z, 0), at.SliceTensor(Z, 1)

    engine("BX_e_i1_k2 = B_k2_i2 X_e_i1_i2", T, tB, tX)
    engine("U1_e_k1_k2 = G_k1_i1 BX_e_i1_k2", U1, tG, T)
    engine("GX_e_i1_k2 = G_k2_i2 X_e_i1_i2", T, tG, tX)
    engine("U2_e_k1_k2 = B_k1_i1 GX_e_i1_k2", U2, tB, T)
    engine("Z_m_e_k1_k2 = D_e_m_n_k1_k2 U_n_e_k1_k2", Z, tD, U)
    U.MoveFromGPU()
    expU = np.stack([np.einsum("ai,bj,eij->eab", G, B, X), np.einsum("ai,bj,eij->eab", B, G, X)])
    assert np.array_equal(U.data, expU)
    expZ = np.einsum("emnab,neab->meab", D, expU)
    Z.MoveFromGPU()
    assert np.array_equal(Z.data, expZ)

    engine("BZ1_e_i2_k1 = B_k2_i2 Z1_e_k1_k2", T, tB, Z1)
    engine("Y_e_i1_i2 = G_k1_i1 BZ1_e_i2_k1", Y, tG, T)
    Y.MoveFromGPU()
    assert np.array_equal(Y.data, np.einsum("ai,bj,eab->eij", G, B, expZ[0]))
    engine("GZ2_e_i2_k1 = G_k2_i2 Z2_e_k1_k2", T, tG, Z2)
    engine("Y_e_i1_i2 = B_k1_i1 GZ2_e_i2_k1", Y, tB, T)
    Y.MoveFromGPU()
    assert np.array_equal(Y.data, np.einsum("ai,bj,eab->eij", B, G, expZ[1]))


def test_2d_stiffness_as_one_multi_kernel_launch_with_aliased_slices(at, engine):
    # Same computation captured as ONE multi-kernel launch: U1/U2 are written under their own names and read
    # back through U, so the variables overlap in memory and the launch must not be fused blindly.
    B, G, X, D = seq((4, 4)), seq((4, 4), scale=0.5), seq((5, 4, 4)), seq((5, 2, 2, 4, 4))
    tB, tG, tX, tD = (to_tensor(at, a) for a in (B, G, X, D))
    T1, T2, U, Z = at.Tensor(5, 4, 4), at.Tensor(5, 4, 4), at.Tensor(2, 5, 4, 4), at.Tensor(2, 5, 4, 4)
    U1, U2 = at.SliceTensor(U, 0), at.SliceTensor(U, 1)
    engine.BeginMultiKernelLaunch()
    engine("BX_e_i1_k2 = B_k2_i2 X_e_i1_i2", T1, tB, tX)
    engine("U1_e_k1_k2 = G_k1_i1 BX_e_i1_k2", U1, tG, T1)
    engine("GX_e_i1_k2 = G_k2_i2 X_e_i1_i2", T2, tG, tX)
    engine("U2_e_k1_k2 = B_k1_i1 GX_e_i1_k2", U2, tB, T2)
    engine("Z_m_e_k1_k2 = D_e_m_n_k1_k2 U_n_e_k1_k2", Z, tD, U)
    engine.EndMultiKernelLaunch()
    Z.MoveFromGPU()
    expU = np.stack([np.einsum("ai,bj,eij->eab", G, B, X), np.einsum("ai,bj,eij->eab", B, G, X)])
    assert np.array_equal(Z.data, np.einsum("emnab,neab->meab", D, expU))


def test_3d_stiffness_twelve_loops(at, engine, checker):
    # unittest/kernel/test_TensorEngine.cpp:437-496 (contraction of 1125 terms: counted-loop path), E reduced to 4
    k = "S_e_i1_i2_i3_j1_j2_j3 = B1_i1_j1_k1_m_n B2_i2_j2_k2_m_n B3_i3_j3_k3_m_n D_e_k1_k2_k3_m_n"
    B1 = seq((5, 5, 5, 3, 3), mod=11)
    B2 = seq((5, 5, 5, 3, 3), mod=7, scale=2.0)
    B3 = seq((5, 5, 5, 3, 3), mod=13, scale=3.0)
    D = seq((4, 5, 5, 5, 3, 3), mod=5, scale=3.5)
    got, expected = run_single(at, engine, checker, k, np.zeros((4, 5, 5, 5, 5, 5, 5)), B1, B2, B3, D)
    assert np.array_equal(got, expected)          # all terms are multiples of 0.5 below 2^53: exact


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i_j = B_e_i_k C_e_k_j", [(37, 16, 16), (37, 16, 16)]),          # the reference's I_b_i_k = TI_b_i_j T_b_j_k, larger
    ("A_e_i_j += B_e_i_k C_e_j_k", [(21, 16, 12), (21, 20, 12)]),         # second factor transposed, rectangular
    ("A_e_j_i -= B_e_k_i C_e_k_j W_e", [(40, 7, 32), (40, 7, 24), (40,)]),   # both transposed, output transposed, a factor per entry
    ("A_e_i_j = C_e_k_j B_e_i_k D_e_i_j", [(14, 9, 11), (14, 13, 9), (14, 13, 11)]),   # pointwise factor on the result
])
def test_products_of_element_matrices_stage_their_operands_in_lds(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel))
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "operands staged in LDS" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes,expect", [
    # 3 x 3 (the reference's unittest/kernel/test_TensorEngine.cpp:292-331 is 2 x 2): one output per lane, 56 entries per workgroup
    ("A_e_i_j = B_e_i_k C_e_k_j", [(1001, 3, 3), (1001, 3, 3)], "56 per workgroup of 256 lanes"),
    ("A_e_i_j -= B_e_k_i C_e_j_k", [(333, 5, 7), (333, 6, 5)], "lanes(i,j)=42 tile()=1"),
    ("A_e_i_j += B_e_i_k C_e_k_l D_e_l_j", [(77, 3, 3), (77, 3, 3), (77, 3, 3)], "operands staged in LDS"),
    # entries of whole lines: staged from 16 outputs on (32 entries per workgroup, ragged end)
    ("A_e_i_j += B_e_i_k C_e_k_j", [(1001, 4, 4), (1001, 4, 4)], "32 per workgroup of 256 lanes"),
    ("A_e_i_j = B_e_i_k C_e_j_k", [(77, 8, 2), (77, 2, 2)], "lanes(i,j)=16 tile()=1"),
    # even extents: both output indices split in two, a 2 x 2 block of outputs per lane
    ("A_e_i_j = B_e_i_k C_e_k_j", [(203, 12, 12), (203, 12, 12)], "lanes(ihi,jhi)=36 tile(ilo,jlo)=4"),
    ("A_e_j_i += B_e_k_i C_e_j_k W_e", [(57, 9, 24), (57, 30, 9), (57,)], "tile(jlo,ilo)=4"),
    # divisible by three only: 3 x 3 blocks; one index split, the other prime
    ("A_e_i_j -= B_e_i_k C_e_j_k", [(45, 9, 10), (45, 15, 10)], "tile(ilo,jlo)=9"),
    ("A_e_i_j = B_e_i_k C_e_k_j D_e_i_j", [(31, 24, 8), (31, 8, 25), (31, 24, 25)], "tile(ilo)=2"),
    # no blocks: one output per lane, several entries per workgroup; rows of odd length are padded in LDS
    ("A_e_i_j = B_e_i_k C_e_k_j", [(203, 11, 11), (203, 11, 11)], "8 per workgroup of 256 lanes"),
    # divisible by five only: blocks of five along one index while a hundred lane items are left per entry
    ("A_e_i_j += B_e_i_k C_e_k_j", [(29, 25, 25), (29, 25, 25)], "lanes(ihi,j)=125 tile(ilo)=5"),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(41, 25, 15), (41, 15, 20)], "lanes(ihi,jhi)=50 tile(ilo,jlo)=10"),
    # larger than 32 x 32: an entry's operands fill most of a workgroup's LDS
    ("A_e_i_j -= B_e_i_k C_e_k_j", [(39, 35, 35), (39, 35, 35)], "lanes(ihi,j)=245 tile(ilo)=5"),
])
def test_products_of_small_element_matrices(at, engine, checker, kernel, shapes, expect):
    rng = np.random.default_rng(len(kernel) + shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert "operands staged in LDS" in src and expect in src
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


PRODUCTS_ON_THE_MATRIX_CORES = [
    # (kernel, shapes of the inputs in the order written): square and rectangular, every combination of layouts,
    # extents that are multiples of 16 and extents that are not, odd tensors, the factors in either order
    ("A_e_i_j = B_e_i_k C_e_k_j", [(67, 64, 64), (67, 64, 64)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(129, 63, 63), (129, 63, 63)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(71, 55, 55), (71, 55, 55)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(64, 53, 53), (64, 53, 53)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(100, 37, 37), (100, 37, 37)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(101, 33, 29), (101, 29, 41)]),
    ("A_e_i_j = B_e_i_k C_e_j_k", [(75, 62, 62), (75, 62, 62)]),
    ("A_e_i_j = B_e_k_i C_e_k_j", [(80, 48, 56), (80, 48, 40)]),
    ("A_e_i_j = B_e_k_i C_e_j_k", [(51, 47, 45), (51, 40, 47)]),
    ("A_e_i_j += B_e_i_k C_e_k_j", [(29, 23, 23), (29, 23, 23)]),
    ("A_e_i_j -= C_e_j_k B_e_i_k", [(90, 45, 20), (90, 37, 20)]),
    ("A_e_i_j += B_e_k_i C_e_k_j", [(1001, 9, 17), (1001, 9, 64)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(333, 19, 128), (333, 128, 8)]),
    ("A_e_i_j -= B_e_i_k C_e_j_k", [(257, 31, 31), (257, 31, 31)]),
    # whole blocks of 16 below 36 x 36
    ("A_e_i_j = B_e_i_k C_e_j_k", [(77, 32, 32), (77, 32, 32)]),
    ("A_e_i_j += B_e_k_i C_e_k_j", [(55, 24, 32), (55, 24, 16)]),
    # extents up to 32 that only three divides
    ("A_e_i_j = B_e_i_k C_e_k_j", [(301, 27, 27), (301, 27, 27)]),
    ("A_e_i_j += B_e_k_i C_e_j_k", [(111, 9, 21), (111, 27, 9)]),
    # tensors of odd length whose last double sits in a 16-byte piece that is not a lane's last one
    ("A_e_i_j = C_e_k_j B_e_k_i", [(129, 93, 11), (129, 93, 49)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(145, 27, 67), (145, 67, 19)]),
    # an element matrix applied to an element vector, rows that are no multiple of four doubles: a single column
    ("A_e_i = B_e_i_j C_e_j", [(1001, 27, 27), (1001, 27)]),
    ("A_e_i += B_e_i_j C_e_j", [(333, 45, 31), (333, 31)]),
    ("A_e_i -= C_e_j B_e_i_j", [(129, 27), (129, 64, 27)]),
    ("A_e_i = B_e_i_j C_e_j", [(177, 125, 63), (177, 63)]),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kernel,shapes", PRODUCTS_ON_THE_MATRIX_CORES)
def test_products_of_element_matrices_on_the_matrix_cores_random(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel) + shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.gpu
@pytest.mark.parametrize("kernel,shapes", PRODUCTS_ON_THE_MATRIX_CORES)
def test_products_of_element_matrices_on_the_matrix_cores_integer_exact(at, engine, checker, kernel, shapes):
    """Integer-valued data: sums in any order are exact, so every entry, row, column and term must be in its place
    (also the ones next to the padding of blocks of 16 rows or columns and of steps of four terms)."""
    rng = np.random.default_rng(7 * len(kernel) + shapes[0][1])
    ins = [rng.integers(-5, 6, s).astype(np.float64) for s in shapes]
    out0 = rng.integers(-5, 6, output_shape(kernel, shapes)).astype(np.float64)
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)


@pytest.mark.gpu
def test_products_of_element_matrices_on_the_matrix_cores_views_and_odd_tensors(at, engine, checker):
    """Factors and results that are slices at odd offsets of larger tensors, and tensors with an odd number of
    doubles (whose last one cannot be read as part of a pair)."""
    rng = np.random.default_rng(99)
    E, n = 65, 19                                           # 65 * 19 * 19 doubles: odd; slices start at odd offsets
    B3, C3, A3 = (rng.integers(-4, 5, (3, E, n, n)).astype(np.float64) for _ in range(3))
    tB, tC, tA = (to_tensor(at, x) for x in (B3, C3, A3))
    for which in (1, 2):
        sB, sC, sA = (at.SliceTensor(t, which) for t in (tB, tC, tA))
        engine("A_e_i_j = B_e_i_k C_e_j_k", sA, sB, sC)
        assert "product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    tA.MoveFromGPU()
    expected = A3.copy()
    for which in (1, 2):
        checker.contract("A_e_i_j = B_e_i_k C_e_j_k", expected[which], np.ascontiguousarray(B3[which]), np.ascontiguousarray(C3[which]))
    assert np.array_equal(tA.data, expected)                # also: nothing outside the slices was touched


TILED_PRODUCTS = [
    # (kernel, shapes of the inputs in the order written): matrices beyond 64 rows or columns or 128 terms per entry, and
    # products without a batch index; every combination of layouts, extents that 16 divides and extents that it does
    # not, tiles with and without padding, more than one tile per entry either way, the factors in either order
    ("A_e_i_j = B_e_i_k C_e_k_j", [(7, 128, 128), (7, 128, 128)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(5, 100, 150), (5, 150, 70)]),
    ("A_e_i_j += B_e_k_i C_e_j_k", [(5, 150, 100), (5, 70, 150)]),
    ("A_e_i_j -= B_e_k_i C_e_k_j", [(3, 17, 65), (3, 17, 129)]),
    ("A_e_i_j = C_e_j_k B_e_i_k", [(3, 33, 64), (3, 200, 64)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(2, 300, 40), (2, 40, 260)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(80, 72, 72), (80, 72, 72)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(130, 125, 125), (130, 125, 125)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(64, 32, 200), (64, 200, 48)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(4, 16, 16), (4, 16, 400)]),
    ("A_i_j = B_i_k C_k_j", [(256, 100), (100, 192)]),
    ("A_i_j += B_k_i C_j_k", [(333, 129), (65, 333)]),
    ("A_i_j = B_i_k C_j_k", [(96, 80), (112, 80)]),
    ("A_i_j -= C_k_j B_i_k", [(77, 301), (515, 77)]),
    # few tiles and a long contracted range: shares of the range per workgroup, partial sums added by a second kernel
    ("A_i_j = B_e_i C_e_j", [(3000, 96), (3000, 100)]),
    ("A_i_j -= B_i_k C_k_j", [(65, 4099), (4099, 96)]),
    ("A_e_i_j += B_e_i_k C_e_k_j", [(3, 70, 1500), (3, 1500, 66)]),
    # ... also products of moderate size (a workgroup takes its chunks one after the other, so few tiles leave most of the
    # device idle): a few shares, one lane per output in the second kernel
    ("A_i_j = B_i_k C_k_j", [(256, 256), (256, 256)]),
    ("A_i_j += B_i_k C_k_j", [(300, 520), (520, 200)]),
    # ... fewer than 16 rows or columns under a long contracted range (most of the matrix instruction is padding; the
    # generic schedule would give the whole range to single lanes)
    ("A_i_j = B_i_k C_k_j", [(8, 3000), (3000, 100)]),
    ("A_i_j -= B_k_i C_j_k", [(5000, 3), (300, 5000)]),
    ("A_i_j += B_i_k C_j_k", [(15, 4001), (15, 4001)]),
    ("A_i_j = C_k_j B_i_k", [(2000, 31), (8, 2000)]),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(3, 8, 1500), (3, 1500, 20)]),
    # ... many shares of few outputs: four and sixteen lanes per output in the second kernel
    ("A_i_j = B_n_i C_n_j", [(20000, 144), (20000, 128)]),
    ("A_i_j -= B_i_k C_k_j", [(64, 60000), (60000, 64)]),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kernel,shapes", TILED_PRODUCTS)
def test_products_of_large_matrices_in_tiles_on_the_matrix_cores_random(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel) + shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "tiled product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.gpu
@pytest.mark.parametrize("kernel,shapes", TILED_PRODUCTS)
def test_products_of_large_matrices_in_tiles_on_the_matrix_cores_integer_exact(at, engine, checker, kernel, shapes):
    """Integer-valued data: sums in any order are exact, so every row, column and term must be in its place (also the
    ones next to the padding of tiles, of blocks of 16 and of chunks of terms)."""
    rng = np.random.default_rng(11 * len(kernel) + shapes[0][1])
    ins = [rng.integers(-5, 6, s).astype(np.float64) for s in shapes]
    out0 = rng.integers(-5, 6, output_shape(kernel, shapes)).astype(np.float64)
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "tiled product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)


@pytest.mark.gpu
def test_products_of_large_matrices_in_tiles_views_and_special_values(at, engine, checker):
    """Factors and results that are slices at odd offsets of larger tensors; and a NaN in an entry's first element,
    the element that stands in for values past the end of a matrix, must stay where it belongs."""
    rng = np.random.default_rng(41)
    E, m, k, n = 3, 81, 37, 70
    B3, C3, A3 = (rng.integers(-4, 5, (3, E) + s).astype(np.float64) for s in ((m, k), (k, n), (m, n)))
    tB, tC, tA = (to_tensor(at, x) for x in (B3, C3, A3))
    for which in (1, 2):
        engine("A_e_i_j = B_e_i_k C_e_k_j", at.SliceTensor(tA, which), at.SliceTensor(tB, which), at.SliceTensor(tC, which))
        assert "tiled product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    tA.MoveFromGPU()
    expected = A3.copy()
    for which in (1, 2):
        expected[which] = np.einsum("eik,ekj->eij", B3[which], C3[which])
    assert np.array_equal(tA.data, expected)                # also: nothing outside the slices was touched
    B = rng.integers(-4, 5, (E, m, k)).astype(np.float64)
    C = rng.integers(-4, 5, (E, k, n)).astype(np.float64)
    B[1, 0, 0] = np.nan
    tB, tC, tA = to_tensor(at, B), to_tensor(at, C), at.Tensor(E, m, n)
    engine("A_e_i_j = B_e_i_k C_e_k_j", tA, tB, tC)
    tA.MoveFromGPU()
    expected = np.einsum("eik,ekj->eij", B, C)
    assert np.isnan(tA.data[1, 0]).all() and np.isnan(tA.data).sum() == n
    assert np.array_equal(np.nan_to_num(tA.data), np.nan_to_num(expected))


@pytest.mark.gpu
def test_large_matrix_product_in_tiles_through_properties(at, engine):
    """A 2 048 x 1 536 x 2 560 product without a batch index (256 tiles, 160 chunks of terms each), too large for the
    checker's loops: (B C) x must equal B (C x) for random x, rows and columns of ones must give the row and column sums,
    and integer-valued factors must give the exact integer product in sampled entries."""
    rng = np.random.default_rng(77)
    m, k, n = 2048, 2560, 1536
    B = rng.integers(-3, 4, (m, k)).astype(np.float64)
    C = rng.integers(-3, 4, (k, n)).astype(np.float64)
    tA, tB, tC = at.Tensor(m, n), to_tensor(at, B), to_tensor(at, C)
    engine("A_i_j = B_i_k C_k_j", tA, tB, tC)
    assert "tiled product schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    tA.MoveFromGPU()
    A = tA.data
    x = rng.integers(-2, 3, (n, 3)).astype(np.float64)
    assert np.array_equal(A @ x, B @ (C @ x))                                   # integers: exact in any order
    y = rng.integers(-2, 3, (3, m)).astype(np.float64)
    assert np.array_equal(y @ A, (y @ B) @ C)
    rows = rng.integers(0, m, 40)
    assert np.array_equal(A[rows], B[rows] @ C)
    # the same with the second factor transposed and accumulation, random data: <= 1e-12 against numpy in sampled rows
    Bf, Cf = rng.uniform(-1, 1, (m, k)), rng.uniform(-1, 1, (n, k))
    A0 = rng.uniform(-1, 1, (m, n))
    tA, tB, tC = to_tensor(at, A0), to_tensor(at, Bf), to_tensor(at, Cf)
    engine("A_i_j += B_i_k C_j_k", tA, tB, tC)
    tA.MoveFromGPU()
    assert rel_err(tA.data[rows], A0[rows] + Bf[rows] @ Cf.T) <= TOL


@pytest.mark.gpu
def test_normal_equations_with_many_columns_share_out_the_rows(at, engine):
    """A_i_j = B_n_i C_n_j with 144 x 128 outputs over 2^17 rows: more blocks than the Gram schedule holds, so tiles with
    the contracted range shared out over 86 workgroups per tile; against numpy, integer data exact, twice in a row
    (the scratch buffer of partial tiles is reused)."""
    rng = np.random.default_rng(78)
    rows, ni, nj = 1 << 17, 144, 128
    B = rng.integers(-3, 4, (rows, ni)).astype(np.float64)
    C = rng.integers(-3, 4, (rows, nj)).astype(np.float64)
    tA, tB, tC = at.Tensor(ni, nj), to_tensor(at, B), to_tensor(at, C)
    expected = B.T @ C
    for _ in range(2):
        engine("A_i_j = B_n_i C_n_j", tA, tB, tC)
        src = engine.GetLastImplementation()
        assert "tiled product schedule" in src and "shares of" in src
        tA.MoveFromGPU()
        assert np.array_equal(tA.data, expected)
    engine("A_i_j -= B_n_i C_n_j", tA, tB, tC)
    tA.MoveFromGPU()
    assert np.array_equal(tA.data, np.zeros((ni, nj)))


def test_product_of_slices_keeps_its_indices(at, engine, checker):
    # operands that are views into larger tensors are not described by split dimensions
    rng = np.random.default_rng(12)
    big = rng.uniform(-1, 1, (2, 50, 12, 12))
    C = rng.uniform(-1, 1, (50, 12, 12))
    tbig, tC, tA = to_tensor(at, big), to_tensor(at, C), at.Tensor(50, 12, 12)
    engine("A_e_i_j = B_e_i_k C_e_k_j", tA, at.SliceTensor(tbig, 1), tC)
    tA.MoveFromGPU()
    src = engine.GetLastImplementation()
    assert "operands staged in LDS" in src and "ihi" not in src
    assert rel_err(tA.data, np.einsum("eik,ekj->eij", big[1], C)) <= TOL


@pytest.mark.parametrize("P,Q,E", [(2, 3, 1001), (4, 5, 203), (3, 4, 77), (8, 10, 5)])
def test_2d_mass_assembly_results_leave_through_an_lds_tile(at, engine, checker, P, Q, E):
    # unittest/kernel/test_TensorEngine.cpp:399-435 at other sizes.  With lanes (i2, j2) / (j1, j2) and a register tile
    # in between, a store instruction would write pieces of a few doubles far apart: the results go to an LDS tile
    # and the workgroup writes the tile out in whole lines (also for the kernel evaluated in two steps).
    k = "M_e_i1_i2_j1_j2=B_k1_i1 B_k1_j1 B_k2_i2 B_k2_j2 D_e_k1_k2"
    rng = np.random.default_rng(P * 100 + Q)
    B = rng.integers(-2, 3, (Q, P)).astype(np.float64)
    D = rng.integers(-3, 4, (E, Q, Q)).astype(np.float64)
    got, expected = run_single(at, engine, checker, k, np.full((E, P, P, P, P), 7.0), B, B, B, B, D)
    assert np.array_equal(got, expected)                      # small integers: exact whatever the order of the sums
    assert np.array_equal(got, np.einsum("ai,aj,bk,bl,eab->eikjl", B, B, B, B, D))
    if (P, Q) in ((2, 3), (4, 5)):
        assert "M->lds+global" in engine.GetLastImplementation()


@pytest.mark.parametrize("order", [1, 4])
def test_d_tensor_construction(at, engine, checker, order):
    # unittest/kernel/test_TensorEngine.cpp:498-590
    rng = np.random.default_rng(order)
    n, E = order + 1, 6
    W, C = rng.uniform(0.5, 1, (E, n, n)), rng.uniform(0.5, 1, (E, n, n))
    J = np.eye(2) + 0.1 * rng.uniform(-1, 1, (E, n, n, 2, 2))
    tJ, Jinv, Jdet = to_tensor(at, J), at.Tensor(E, n, n, 2, 2), at.Tensor(E, n, n)
    engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
    Jinv.MoveFromGPU()
    Jdet.MoveFromGPU()
    ji, jd = Jinv.data.copy(), Jdet.data.copy()
    got, expected = run_single(at, engine, checker,
                               "D_e_m_n_k1_k2 = W_e_k1_k2 C_e_k1_k2 Jdet_e_k1_k2 Jinv_e_k1_k2_m_j Jinv_e_k1_k2_n_j",
                               np.zeros((E, 2, 2, n, n)), W, C, jd, ji, ji)
    assert rel_err(got, expected) <= TOL
    assert rel_err(got, np.einsum("eab,eab,eab,eabmj,eabnj->emnab", W, C, jd, ji, ji)) <= TOL


@pytest.mark.parametrize("m", [1, 2, 3])
def test_batch_matrix_inverse_and_determinant(at, engine, checker, m):
    # unittest/kernel/test_TensorEngine.cpp:594-706; non-symmetric matrices on purpose
    rng = np.random.default_rng(m)
    A = np.eye(m) + 0.2 * rng.uniform(-1, 1, (37, 5, m, m))
    tA, Ainv, Adet, Ainv2, Adet2 = to_tensor(at, A), at.Tensor(37, 5, m, m), at.Tensor(37, 5), at.Tensor(37, 5, m, m), at.Tensor(37, 5)
    engine.BatchMatrixInverse(Ainv, tA)
    engine.BatchMatrixDet(Adet, tA)
    engine.BatchMatrixInvDet(Ainv2, Adet2, tA)
    for t in (Ainv, Adet, Ainv2, Adet2):
        t.MoveFromGPU()
    ri, rd = checker.batch_matrix_inv_det(A)
    assert np.array_equal(Ainv.data, ri) and np.array_equal(Ainv2.data, ri)      # bit for bit
    assert np.array_equal(Adet.data, rd) and np.array_equal(Adet2.data, rd)
    # invariants: A * Ainv^T = I for 3x3 (the reference's layout), A * Ainv = I otherwise; det(A) det(Ainv) = 1
    prod = np.einsum("...ij,...kj->...ik", A, Ainv.data) if m == 3 else np.einsum("...ij,...jk->...ik", A, Ainv.data)
    assert np.abs(prod - np.eye(m)).max() < 1e-13
    # I_b_i_k = TI_b_i_j T_b_j_k through the engine, as the reference's test does
    I = at.Tensor(37 * 5, m, m)
    Ainv.Reshape(37 * 5, m, m)
    tA.Reshape(37 * 5, m, m)
    if m == 3:
        engine("I_b_i_k = TI_b_j_i T_b_j_k", I, Ainv, tA)
    else:
        engine("I_b_i_k = TI_b_i_j T_b_j_k", I, Ainv, tA)
    I.MoveFromGPU()
    assert np.abs(I.data - np.eye(m)).max() < 1e-13


def test_batch_matrix_shape_asserts(at, engine):
    # unittest/kernel/test_TensorEngine.cpp:600-612
    A4, A3, B3, d = at.Tensor(5, 4, 4), at.Tensor(5, 3, 3), at.Tensor(6, 3, 3), at.Tensor(5)
    for t in (A4, A3, B3):
        t.Set(1.0)
    with pytest.raises(at.AcroError):
        engine.BatchMatrixInverse(at.Tensor(5, 4, 4), A4)        # larger than 3x3
    with pytest.raises(at.AcroError):
        engine.BatchMatrixInverse(B3, A3)                        # batch mismatch
    with pytest.raises(at.AcroError):
        engine.BatchMatrixDet(at.Tensor(6), A3)
    with pytest.raises(at.AcroError):
        engine.BatchMatrixDet(d, at.Tensor(5, 3, 2))             # not square
    with pytest.raises(at.AcroError):
        engine.BatchMatrixInvDet(at.Tensor(5, 3, 3), at.Tensor(5, 1), A3)


def test_batch_matrix_ragged_batch_sizes(at, engine, checker):
    for n in (1, 63, 64, 65, 255, 256, 257, 1000):
        rng = np.random.default_rng(n)
        A = np.eye(3) + 0.1 * rng.uniform(-1, 1, (n, 3, 3))
        tA, Ainv, Adet = to_tensor(at, A), at.Tensor(n, 3, 3), at.Tensor(n)
        engine.BatchMatrixInvDet(Ainv, Adet, tA)
        Ainv.MoveFromGPU()
        Adet.MoveFromGPU()
        ri, rd = checker.batch_matrix_inv_det(A)
        assert np.array_equal(Ainv.data, ri) and np.array_equal(Adet.data, rd)


def test_scatter_and_sum_gather(at, engine, checker):
    # unittest/kernel/test_TensorEngine.cpp:708-745: the 8 -> 6 map
    M = at.IndexMapping(6, 8)
    M.map[:] = [0, 1, 2, 3, 4, 5, 1, 3]
    src = to_tensor(at, np.arange(6, dtype=np.float64) * 10)
    out = at.Tensor(8)
    engine.FlatIndexedScatter(out, src, M)
    out.MoveFromGPU()
    assert np.array_equal(out.data, [0, 10, 20, 30, 40, 50, 10, 30])
    vals = to_tensor(at, np.arange(1, 9, dtype=np.float64))
    acc = at.Tensor(6)
    engine.FlatIndexedSumGather(acc, vals, M)
    acc.MoveFromGPU()
    assert np.array_equal(acc.data, [1, 9, 3, 12, 5, 6])
    with pytest.raises(at.AcroError):
        engine.FlatIndexedScatter(at.Tensor(7), src, M)
    with pytest.raises(at.AcroError):
        engine.FlatIndexedSumGather(at.Tensor(5), vals, M)


def test_sum_gather_large_random_map_bit_exact(at, engine, checker):
    rng = np.random.default_rng(8)
    domain, rsize = 5000, 40000
    M = at.IndexMapping(domain, rsize)
    M.map[:] = rng.integers(0, domain - 7, rsize)              # the last domain entries have no preimage
    vals = rng.uniform(-1, 1, rsize)
    acc = at.Tensor(domain)
    engine.FlatIndexedSumGather(acc, to_tensor(at, vals), M)
    acc.MoveFromGPU()
    assert np.array_equal(acc.data, checker.sum_gather(vals, M.map, domain))
    src = rng.uniform(-1, 1, domain)
    out = at.Tensor(rsize)
    engine.FlatIndexedScatter(out, to_tensor(at, src), M)
    out.MoveFromGPU()
    assert np.array_equal(out.data, checker.scatter(src, M.map))


@pytest.mark.parametrize("domain,rsize,skew", [(1, 9001, 0), (1030, 3, 0), (2500, 70001, 3), (4099, 4099, 0)])
def test_scatter_and_sum_gather_ragged_maps_bit_exact(at, engine, checker, domain, rsize, skew):
    # rows of the inverse map from empty to tens of thousands of entries (longer than one staging chunk), domain and
    # range sizes that are not multiples of the workgroup or vector width
    rng = np.random.default_rng(domain + rsize)
    M = at.IndexMapping(domain, rsize)
    m = rng.integers(0, domain, rsize)
    if skew:
        m[rng.uniform(size=rsize) < 0.6] = domain // skew          # one very long row
    M.map[:] = m
    vals = rng.uniform(-1, 1, rsize)
    acc = at.Tensor(domain)
    acc.Set(99.0)                                                  # must be overwritten, also where no entry maps
    engine.FlatIndexedSumGather(acc, to_tensor(at, vals), M)
    acc.MoveFromGPU()
    assert np.array_equal(acc.data, checker.sum_gather(vals, M.map, domain))
    src = rng.uniform(-1, 1, domain)
    out = at.Tensor(rsize)
    engine.FlatIndexedScatter(out, to_tensor(at, src), M)
    out.MoveFromGPU()
    assert np.array_equal(out.data, checker.scatter(src, M.map))


def test_scatter_into_a_slice_that_is_not_vector_aligned(at, engine, checker):
    rng = np.random.default_rng(77)
    domain, rsize = 300, 1001                                       # slices start at odd multiples of 8 bytes
    M = at.IndexMapping(domain, rsize)
    M.map[:] = rng.integers(0, domain, rsize)
    src = rng.uniform(-1, 1, domain)
    parent = at.Tensor(3, rsize)
    parent.Set(-5.0)
    parent.MoveToGPU()      # an output that is still on the host is switched, not copied (kernel/TensorEngine.cpp:692-699)
    out = at.SliceTensor(parent, 1)
    engine.FlatIndexedScatter(out, to_tensor(at, src), M)
    parent.MoveFromGPU()
    assert np.array_equal(parent.data[1], checker.scatter(src, M.map))
    assert np.all(parent.data[0] == -5.0) and np.all(parent.data[2] == -5.0)


def test_few_batch_entries_with_many_work_items_spread_over_workgroups(at, engine, checker):
    # 12 batch entries (the largest output index) x 4 950 work items: one workgroup per entry would use 12 of 256
    # CUs, so the passes of the item loop become a second grid dimension
    rng = np.random.default_rng(21)
    B, C = rng.uniform(-1, 1, (12, 11, 10, 9, 5, 6)), rng.uniform(-1, 1, 6)
    k = "A_a_b_c_d_f = B_a_b_c_d_f_k C_k"
    got, expected = run_single(at, engine, checker, k, np.zeros((12, 11, 10, 9, 5)), B, C)
    assert "blockIdx.y" in engine.GetLastImplementation()
    assert rel_err(got, expected) <= TOL
    got, expected = run_single(at, engine, checker, k.replace(" = ", " += "), rng.uniform(-1, 1, (12, 11, 10, 9, 5)), B, C)
    assert rel_err(got, expected) <= TOL


def test_get_implementation_returns_hip_source(at, engine):
    A, B = at.Tensor(8, 3), at.Tensor(8, 3)
    src = engine.GetImplementation("A_e_i = B_e_i", A, B)
    assert "__global__" in src and "A_e_i = B_e_i" in src


def test_partially_written_parent_is_read_back_from_device_memory(at, engine):
    # U0 is produced inside the launch, U1 keeps what it held before; the whole-U read must see both
    rng = np.random.default_rng(77)
    E = 13
    X, G, D = rng.uniform(-1, 1, (E, 4)), rng.uniform(-1, 1, (5, 4)), rng.uniform(-1, 1, (E, 5, 2, 2))
    U_init = rng.uniform(-1, 1, (2, E, 5))
    for transient in (False, True):
        tX, tG, tD, U, Z = to_tensor(at, X), to_tensor(at, G), to_tensor(at, D), to_tensor(at, U_init), at.Tensor(2, E, 5)
        U.SetTransient(transient)
        U0 = at.SliceTensor(U, 0)
        engine.BeginMultiKernelLaunch()
        engine("U0_e_q = G_q_i X_e_i", U0, tG, tX)
        engine("Z_m_e_q = D_e_q_m_n U_n_e_q", Z, tD, U)
        engine.EndMultiKernelLaunch()
        Z.MoveFromGPU()
        expU = U_init.copy()
        expU[0] = X @ G.T
        assert rel_err(Z.data, np.einsum("eqmn,neq->meq", D, expU)) <= TOL


def test_slice_of_a_slice_inside_a_fused_launch(at, engine):
    rng = np.random.default_rng(78)
    E = 9
    P = at.Tensor(2, 3, E, 4)
    P.data[...] = rng.uniform(-1, 1, (2, 3, E, 4))
    before = P.data.copy()
    S1 = at.SliceTensor(P, 1)            # [3, E, 4]
    S12 = at.SliceTensor(S1, 2)          # [E, 4]  = P[1, 2]
    A, R = to_tensor(at, rng.uniform(-1, 1, (E, 4))), at.Tensor(3, E)
    engine.BeginMultiKernelLaunch()
    engine("V_e_i = A_e_i", S12, A)
    engine("R_a_e = W_a_e_i", R, S1)
    engine.EndMultiKernelLaunch()
    R.MoveFromGPU()
    P.MoveFromGPU()
    expected = before.copy()
    expected[1, 2] = A.data
    assert np.array_equal(P.data, expected)
    assert rel_err(R.data, expected[1].sum(axis=2)) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i = B_i_j X_e_k_j W_e_k", [(64, 64), (1000, 2, 64), (1000, 2)]),   # B staged in LDS, 16 entries per workgroup, ragged end
    ("A_e_i = B_i_j X_e_k_j W_e_k", [(40, 24), (3, 2, 24), (3, 2)]),      # fewer entries than a workgroup would take
    ("A_e_i_k = B_i_j C_k_l X_e_j_l", [(12, 10), (9, 11), (77, 10, 11)]),   # two staged tables, reordered into steps
    ("A_e_i_k = B_e_i_j C_e_j_k", [(1001, 4, 4), (1001, 4, 4)]), # one output per lane
    ("A_e_i_k = B_e_i_j C_e_j_k", [(333, 3, 3), (333, 3, 3)]),
    ("A_e_i = B_e_i_j C_e_j", [(515, 8, 8), (515, 8)]),          # one lane per row
])
def test_kernels_whose_schedule_follows_the_memory_access_pattern(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel) + shapes[-1][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, np.zeros(output_shape(kernel, shapes)), *ins)
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e = B_e_i C_e_i", [(1003, 16), (1003, 16)]),             # 16 lanes per entry
    ("A_e += B_e_i C_e_i", [(77, 67), (77, 67)]),                # 16 lanes, 67 terms: the first three take five (short odd rows: through LDS)
    ("A_e -= B_e_n", [(301, 1000)]),                             # 64 lanes per entry
    ("A_e = B_e_i_j C_j_i", [(130, 5, 13), (13, 5)]),            # two contraction indices, one operand transposed
    ("A_e = B_e_i_j C_e_i_j D_j", [(64, 6, 4), (64, 6, 4), (4,)]),
    ("A_e = B_i_e_j C_e_j", [(3, 50, 11), (50, 11)]),            # batch index in the middle of an operand
    ("A_e_i = B_e_i_j C_e_j", [(203, 16, 16), (203, 16)]),       # element matrix times element vector: 4 lanes per row
    ("A_e_i += B_e_i_j C_e_j", [(35, 20, 20), (35, 20)]),        # 20 terms over 4 lanes (rows of odd length: two steps through LDS)
    ("A_e_i = B_e_i_j C_e_j", [(9, 64, 64), (9, 64)]),           # 16 lanes per row, four passes per entry
    ("A_e_i -= B_e_i_j C_e_j D_e_i", [(130, 100, 100), (130, 100), (130, 100)]),   # more than 64 rows of 32 terms and more: 16 lanes per row
    ("A_e_i = B_e_i_j C_j", [(1030, 300, 33), (33,)]),           # ... rows of odd length
    ("A_e_i_k = B_e_i_k_n", [(21, 3, 5, 100)]),                  # two lane indices next to the shared contraction
    ("A_e -= B_e_i_j C_i D_j", [(1001, 8, 8), (8,), (8,)]),      # bilinear form: pairs of terms along j, C_i once per pair
    ("A_e_i = B_e_i_j_k C_e_j D_e_k", [(203, 8, 8, 8), (203, 8), (203, 8)]),
    ("A_e += B_e_i_j C_e_i D_e_j", [(77, 5, 6), (77, 5), (77, 6)]),
])
def test_one_output_per_batch_entry_shares_the_contraction_between_lanes(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel) + shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "contraction shared by" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected       # the checker adds for "-=", as the reference's interpreter does
    assert rel_err(got, expected) <= TOL
    again, _ = run_single(at, engine, checker, kernel, out0, *ins)
    assert np.array_equal(got, again)                            # fixed order of the lane exchanges: reproducible


@pytest.mark.parametrize("kernel,shapes,out", [
    ("S_i = A_i_n", [(64, 70001)], (64,)),                       # four rows per workgroup, 64 lanes along each
    ("S_i += A_i_n B_n", [(6, 9000), (9000,)], (6,)),            # last group of outputs half empty
    ("S_i_j = A_i_j_n", [(5, 7, 4099)], (5, 7)),
    ("S_i = A_i_m_n B_m", [(9, 3, 3001), (3,)], (9,)),           # two contraction indices
])
def test_split_contraction_of_few_long_rows(at, engine, checker, kernel, shapes, out):
    rng = np.random.default_rng(shapes[0][-1])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, out)
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "64 adjacent lanes along each" in engine.GetLastImplementation()
    assert rel_err(got, expected) <= TOL
    again, _ = run_single(at, engine, checker, kernel, out0, *ins)
    assert np.array_equal(got, again)


@pytest.mark.parametrize("kernel,shape", [
    ("A_i_j = B_j_i", (70, 100)),                    # ragged tiles on both sides
    ("A_i_j += B_j_i", (64, 32)),
    ("A_i_e_j -= B_j_e_i", (70, 3, 100)),            # a dimension in between
    ("A_e_i_j = B_e_j_i", (5, 128, 160)),            # batched, matrices larger than the caches hold per entry
    ("A_e_i_j -= B_e_j_i", (11, 32, 32)),            # ... and small ones that fill the tiles
    ("A_j_k_i = B_i_k_j", (33, 2, 45)),
    ("A_k_j_i_l = B_l_i_k_j", (32, 37, 3, 41)),      # fastest dimensions l and j, two more in other places
    ("A_i_j = B_j_i", (1000, 16)),                   # one side short: tiles of 16 x 64 entries
    ("A_i_j -= B_j_i", (9, 2003)),                   # ... of 64 x 16, the short side ragged (9 of 16)
    ("A_e_i_j = B_e_j_i", (3, 300, 8)),              # ... of 8 x 128, batched
    ("A_i_e_j += B_j_e_i", (24, 2, 257)),            # 24 of 32 on one side
])
def test_permutations_with_long_fastest_dimensions_go_through_lds_tiles(at, engine, checker, kernel, shape):
    rng = np.random.default_rng(sum(shape))
    B = rng.uniform(-1, 1, shape)
    out0 = rng.uniform(-1, 1, output_shape(kernel, [shape]))
    got, expected = run_single(at, engine, checker, kernel, out0, B)
    assert "transpose schedule" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)             # moves (and one addition): bit for bit


@pytest.mark.parametrize("kernel,shape", [
    ("A_e_i_j = B_e_j_i", (5, 40, 50)),              # tiles of 32 x 32 would be filled badly
    ("A_e_i_j += B_e_j_i", (7, 64, 64)),
    ("A_e_f_i_j -= B_e_f_j_i", (3, 2, 100, 100)),
])
def test_small_matrices_per_entry_are_transposed_by_a_lane_per_element(at, engine, checker, kernel, shape):
    rng = np.random.default_rng(sum(shape))
    B = rng.uniform(-1, 1, shape)
    out0 = rng.uniform(-1, 1, output_shape(kernel, [shape]))
    got, expected = run_single(at, engine, checker, kernel, out0, B)
    assert "transpose schedule" not in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i = B_i_j X_e_j", [(64, 64), (1000, 64)]),
    ("A_e_i -= B_i_j X_e_j", [(40, 30), (1001, 30)]),                     # ragged: 1001 entries, rows of 30
    ("A_e_i += X_e_j B_i_j", [(20, 17), (23, 17)]),                       # operands the other way round, 23 entries
    ("A_e_i1_i2 = B_i1_i2_j1_j2 X_e_j1_j2", [(5, 6, 4, 7), (77, 4, 7)]),  # several row and column indices
    ("A_e_i = B_i_j X_e_j", [(1000, 4), (9, 4)]),                         # 1000 rows for 9 entries: not this schedule
    # rows a multiple of 16, columns a multiple of 8: nothing to pad for the FP64 matrix cores
    ("A_e_i -= B_i_j X_e_j", [(48, 40), (1001, 40)]),                     # ragged: 9 entries in the last trip
    ("A_e_i += X_e_j B_i_j", [(16, 16), (23, 16)]),                       # operands the other way round, two trips
    ("A_e_i = B_i_j X_e_j", [(32, 24), (4096, 24)]),                      # whole trips only
    ("A_e_i = B_i_j X_e_j", [(16, 16), (40007, 16)]),                     # more trips than wavefronts
    ("A_e_i = B_i_j X_e_j", [(16, 256), (300, 256)]),                     # 64 terms steps, one output tile
    ("A_e_i = B_i_j X_e_j", [(256, 16), (300, 16)]),                      # 16 output tiles
    ("A_e_i = B_i_j X_e_j", [(17, 240), (300, 240)]),                     # padded to 32 x 240: 60 KB of LDS
    ("A_e_i1_i2 -= B_i1_i2_j1_j2 X_e_j1_j2", [(8, 6, 4, 10), (77, 4, 10)]),
    ("A_e_i = B_j_i X_e_j", [(40, 48), (1001, 40)]),                      # the operator stored transposed
    ("A_e_q_i += B_j_i X_e_q_j", [(24, 32), (100, 7, 24)]),               # 700 entries numbered by two indices
    ("A_e_q_i = B_i_j X_e_q_j", [(30, 20), (100, 7, 20)]),                # padded to 32 x 24
    ("A_e_i = B_j_i X_e_j", [(33, 17), (500, 33)]),                       # odd row length: 8-byte loads, padded to 32 x 36
    # small operators: with vectors of even length from 16 rows or 16 columns on, with odd length from 16 columns on
    ("A_e_i = B_i_j X_e_j", [(16, 8), (5000, 8)]),
    ("A_e_i -= B_i_j X_e_j", [(32, 4), (5001, 4)]),
    ("A_e_i = B_i_j X_e_j", [(8, 8), (5000, 8)]),
    ("A_e_i -= B_i_j X_e_j", [(8, 4), (5001, 4)]),
    ("A_e_i += B_i_j X_e_j", [(10, 10), (777, 10)]),
    ("A_e_i = B_i_j X_e_j", [(3, 27), (900, 27)]),
    ("A_e_i_k = B_e_i_j C_j_k", [(600, 8, 8), (8, 8)]),                   # entries (e, i), operator stored transposed
    ("A_e_i = B_i_j X_e_j", [(9, 9), (5000, 9)]),
    ("A_e_i = B_i_j X_e_j", [(4, 8), (5000, 8)]),                         # four rows of short vectors: not this schedule
    # two to four rows applied to vectors of 16 values and more (a gradient at a point)
    ("A_e_i = B_i_j X_e_j", [(3, 32), (5003, 32)]),
    ("A_e_i += B_i_j X_e_j", [(4, 64), (1001, 64)]),
    ("A_e_i -= B_j_i X_e_j", [(16, 2), (2000, 16)]),                      # the operator stored transposed
    ("A_e_d = D_d_i X_e_i", [(3, 100), (700, 100)]),
    ("A_e_i = B_i_j X_e_j", [(7, 9), (5000, 9)]),                         # odd and short: not this schedule
])
def test_dense_operator_applied_to_every_entry(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(shapes[0][0])
    if kernel.startswith("A_e_i += X"):
        shapes = [shapes[1], shapes[0]]
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    if kernel == "A_e_i_k = B_e_i_j C_j_k":
        rows, cols = 8, 8
    else:
        operator = ins[1] if kernel.startswith("A_e_i += X") else ins[0]
        lead = 2 if "_q_" in kernel else 1
        rows = int(np.prod(out0.shape[lead:]))
        cols = operator.size // rows
    # (vectors of even length: from 16 columns on with two rows and more, below that from 16 rows on; below 16 x 16 the
    # generic schedule is as fast or faster)
    chosen = ((rows >= 2 and cols >= 16) or (rows >= 16 and cols >= 4)) if cols % 2 == 0 else (cols >= 16 or (cols >= 9 and rows >= 8))
    chosen = chosen and shapes[0] != (1000, 4)           # (there the batch index is i, which the operator carries)
    assert ("operator schedule on the FP64 matrix cores" in engine.GetLastImplementation()) == chosen
    needs_padding = rows % 16 != 0 or cols % (8 if cols % 2 == 0 else 4) != 0
    assert ("padded" in engine.GetLastImplementation()) == (chosen and needs_padding)
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes,expect", [
    # rows that 16 does not divide: the 16 entries of a trip leave through LDS as one contiguous range
    ("A_e_i = B_i_j X_e_j", [(81, 8), (1003, 8)], "results written out through LDS"),
    ("A_e_i -= B_i_j X_e_j W_e R_e_i", [(27, 12), (999, 12), (999,), (999, 27)], "results written out through LDS"),
    ("A_e_i += B_j_i X_e_j", [(8, 125), (2001, 8)], "__shared__ double stage[4000]"),      # 8 entries at a time
    ("A_e_i = B_i_j X_e_j", [(250, 16), (517, 16)], "left < 4 ? left : 4"),                 # 4 at a time
    # too large for LDS: blocks of rows, one launch each (the gradient at the 64 points of an element)
    ("G_e_d_q = D_d_q_i X_e_i", [(3, 64, 64), (1001, 64)], "rows 128 - 191 of the 192 x 64 operator"),
    ("A_e_i -= B_j_i X_e_j W_e R_i", [(125, 375), (403, 125), (403,), (375,)], "rows 320 - 374 of the 375 x 125 operator (stored transposed)"),
    ("A_e_i += X_e_j B_i_j D_e_j", [(1500, 30), (1000, 30), (1500, 30)], "rows 768 - 999 of the 1000 x 30 operator"),
    # one shared factor of 4 097 to 8 192 entries and at most 96 columns: the operator schedule before the tiled product
    ("A_e_i = B_i_j X_e_j", [(125, 64), (1003, 64)], "rows 0 - 124 of the 125 x 64 operator"),
    ("A_e_i += B_j_i X_e_j", [(48, 96), (777, 48)], "rows 0 - 95 of the 96 x 48 operator (stored transposed)"),
    ("A_e_i -= B_i_j X_e_j", [(80, 60), (2001, 60)], "rows 0 - 79 of the 80 x 60 operator"),
    # the batch index second among the indices that number the entries
    ("A_i_e_j -= B_i_e_k C_k_j W_i_e", [(8, 501, 16), (16, 12), (8, 501)], "4008 entries"),
])
def test_dense_operators_with_odd_rows_or_too_large_for_lds(at, engine, checker, kernel, shapes, expect):
    rng = np.random.default_rng(shapes[0][0] + len(kernel))
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert "operator schedule on the FP64 matrix cores" in src and expect in src
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i = B_i_j X_e_j W_e", [(64, 64), (1000, 64), (1000,)]),                    # one factor per entry
    ("A_e_i += B_i_j X_e_j W_e", [(40, 24), (43, 24), (43,)]),                       # three trips, the last with 11 entries
    ("A_e_k = B_k_i X_e_i D_e_k", [(12, 10), (5003, 10), (5003, 12)]),               # interpolate, then weights per output
    ("A_e_i = B_k_i U_e_k D_e_k", [(12, 10), (5003, 12), (5003, 12)]),               # weights per element, transposed operator
    ("A_e_i -= B_i_j X_e_j W_e D_e_j R_i F_e_i C_j", [(10, 12), (1000, 12), (1000,), (1000, 12), (10,), (1000, 10), (12,)]),
    ("A_e_i = B_i_j X_e_j D_e_j C_j W_e", [(20, 17), (777, 17), (777, 17), (17,), (777,)]),   # odd length: 8-byte loads
    ("A_e_q_i = W_e_q B_i_j X_e_q_j", [(601, 3), (16, 8), (601, 3, 8)]),            # the factor first, two entry indices
])
def test_dense_operator_with_pointwise_factors(at, engine, checker, monkeypatch, kernel, shapes):
    """Factors beside the operator and the vectors: the result is scaled per entry, per output or per row as it is
    stored, the vectors per element or per column as they are loaded (reference semantics: one product per term)."""
    monkeypatch.setenv("ACRO_HIP_OPERATOR_SMALL", "-1")   # (operators below 16 x 16 on their own: brought here as a group would)
    rng = np.random.default_rng(len(kernel) + shapes[1][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "operator schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i = B_i_j X_e_j", [(64, 64), (999, 64)]),
    ("A_e_i -= B_i_j X_e_j", [(40, 30), (1003, 30)]),
    ("A_e_q_i += B_i_j X_e_q_j", [(30, 20), (101, 7, 20)]),
])
def test_dense_operator_through_scalar_loads(at, engine, checker, monkeypatch, kernel, shapes):
    """The variant of the operator schedule that does without the matrix cores."""
    monkeypatch.setenv("ACRO_HIP_OPERATOR_MFMA", "-1")
    rng = np.random.default_rng(shapes[1][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "a lane keeps its row for 4 entries" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_i_e = B_i_j X_j_e", [(64, 64), (64, 1000)]),                                 # 16 entries per trip
    ("A_i_e -= B_i_j X_j_e", [(30, 27), (27, 1002)]),                                # 32 per trip, ragged end, padded to 32 x 28
    ("A_i_e += B_j_i X_j_e", [(27, 30), (27, 1001)]),                                # odd number of entries: one per lane
    ("A_i1_i2_e_q = X_j_e_q B_i1_i2_j", [(40, 7, 9), (6, 5, 40)]),                   # 63 entries numbered by two indices
    ("A_i_e -= B_i_j X_j_e W_e D_j_e R_i F_i_e C_j", [(30, 27), (27, 1002), (1002,), (27, 1002), (30,), (30, 1002), (27,)]),
    ("A_k_e = B_k_i X_i_e D_k_e", [(24, 22), (22, 5003), (24, 5003)]),
    ("A_i_e = B_i_j X_j_e", [(16, 16), (16, 3000)]),                                 # small operator: not this schedule
])
def test_dense_operator_with_the_entries_as_the_fastest_dimension(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel) + shapes[1][-1])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert ("matrix cores, entries fastest" in engine.GetLastImplementation()) == (shapes[0] != (16, 16))
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("nq,nd,entries,transient", [(32, 27, 1003, True), (32, 27, 1003, False), (64, 64, 517, True), (8, 8, 1000, True),
                                                     (30, 27, 1024, True), (27, 64, 700, True), (64, 27, 5000, True), (33, 17, 999, True),
                                                     (8, 8, 1000, False), (12, 10, 3001, True), (16, 16, 4096, True)])
def test_dense_operator_applied_and_applied_back_in_one_capture(at, engine, checker, nq, nd, entries, transient):
    """Y = Bt (D o (B X)) recorded as two kernels.  Both products run in one matrix-core kernel, the intermediate
    handed over through LDS (and stored unless it is transient); operators too large for that run as one
    matrix-core launch per kernel."""
    rng = np.random.default_rng(nq * nd + entries)
    B, X, D = rng.uniform(-1, 1, (nq, nd)), rng.uniform(-1, 1, (entries, nd)), rng.uniform(0.5, 1.5, (entries, nq))
    Y0 = rng.uniform(-1, 1, (entries, nd))
    tB, tX, tD, tY, tU = to_tensor(at, B), to_tensor(at, X), to_tensor(at, D), to_tensor(at, Y0), at.Tensor(entries, nq)
    tU.SetTransient(transient)
    print("operator chain", nq, nd, entries, transient, flush=True)
    engine.BeginMultiKernelLaunch()
    engine("U_e_k = B_k_j X_e_j D_e_k", tU, tB, tX, tD)
    engine("Y_e_i += B_k_i U_e_k", tY, tB, tU)
    engine.EndMultiKernelLaunch()
    src = engine.GetLastImplementation()
    cols = -(-nd // 8) * 8 if nd % 2 == 0 else -(-nd // 4) * 4
    fits = (-(-nq // 16) * 16 * cols + -(-nd // 16) * 16 * -(-nq // 4) * 4 + 64 * (nq + 1)) * 8 <= 65536
    if fits:
        assert src.count("__global__") == 1 and "applied to the first result on chip" in src
    elif nq * nd >= 512:
        assert src.count("operator schedule on the FP64 matrix cores") == 2
    else:
        assert "operator schedule" not in src
    tY.MoveFromGPU()
    U = np.zeros((entries, nq))
    checker.contract("U_e_k = B_k_j X_e_j D_e_k", U, B, X, D)
    expected = Y0.copy()
    checker.contract("Y_e_i += B_k_i U_e_k", expected, B, U)
    assert rel_err(tY.data, expected) <= TOL
    if not transient:
        tU.MoveFromGPU()
        assert rel_err(tU.data, U) <= TOL


@pytest.mark.parametrize("nq,nd,entries,three", [(32, 27, 1003, True), (64, 27, 700, True), (12, 10, 2001, True), (64, 64, 300, True), (32, 27, 1003, False)])
def test_pointwise_kernels_between_dense_operators_are_folded_into_them(at, engine, checker, nq, nd, entries, three):
    """U = B X, V = U o D, Y = Bt V written as three kernels (or the first two alone) with transient intermediates:
    the pointwise kernel becomes a factor of the operator kernel before it."""
    rng = np.random.default_rng(nq + nd + entries)
    B, X, D = rng.uniform(-1, 1, (nq, nd)), rng.uniform(-1, 1, (entries, nd)), rng.uniform(0.5, 1.5, (entries, nq))
    tB, tX, tD = to_tensor(at, B), to_tensor(at, X), to_tensor(at, D)
    tU, tV, tY = at.Tensor(entries, nq), at.Tensor(entries, nq), at.Tensor(entries, nd)
    tU.SetTransient(True)
    tV.SetTransient(three)
    print("folded chain", nq, nd, entries, three, flush=True)
    engine.BeginMultiKernelLaunch()
    engine("U_e_k = B_k_j X_e_j", tU, tB, tX)
    engine("V_e_k = D_e_k U_e_k", tV, tD, tU)
    if three:
        engine("Y_e_i = B_k_i V_e_k", tY, tB, tV)
    engine.EndMultiKernelLaunch()
    src = engine.GetLastImplementation()
    assert "[0] U_e_k = B_k_j X_e_j ; V_e_k = D_e_k U_e_k" in src
    V = np.zeros((entries, nq))
    checker.contract("V_e_k = B_k_j X_e_j D_e_k", V, B, X, D)
    if three:
        assert ("applied to the first result on chip" in src) == (nq < 64 or nd < 64)
        expected = np.zeros((entries, nd))
        checker.contract("Y_e_i = B_k_i V_e_k", expected, B, V)
        tY.MoveFromGPU()
        assert rel_err(tY.data, expected) <= TOL
    else:
        assert src.count("__global__") == 1
        tV.MoveFromGPU()
        assert rel_err(tV.data, V) <= TOL


@pytest.mark.parametrize("nq,nd,entries", [(30, 27, 1003), (64, 27, 512), (12, 10, 2001)])
def test_second_operator_with_factors_on_the_intermediate(at, engine, checker, nq, nd, entries):
    """U = B X, then Y = Bt (U o D o C) with the weights written into the second kernel: they are applied as the
    intermediate is read back from LDS."""
    rng = np.random.default_rng(nq * nd + entries)
    B, X = rng.uniform(-1, 1, (nq, nd)), rng.uniform(-1, 1, (entries, nd))
    D, C, W = rng.uniform(0.5, 1.5, (entries, nq)), rng.uniform(0.5, 1.5, nq), rng.uniform(0.5, 1.5, entries)
    Y0 = rng.uniform(-1, 1, (entries, nd))
    tB, tX, tD, tC, tW, tY = (to_tensor(at, a) for a in (B, X, D, C, W, Y0))
    tU = at.Tensor(entries, nq)
    tU.SetTransient(True)
    print("operator pair with factors", nq, nd, entries, flush=True)
    engine.BeginMultiKernelLaunch()
    engine("U_e_k = B_k_j X_e_j", tU, tB, tX)
    engine("Y_e_i -= B_k_i U_e_k D_e_k C_k W_e", tY, tB, tU, tD, tC, tW)
    engine.EndMultiKernelLaunch()
    assert "applied to the first result on chip" in engine.GetLastImplementation()
    U = np.zeros((entries, nq))
    checker.contract("U_e_k = B_k_j X_e_j", U, B, X)
    expected = Y0.copy()
    checker.contract("Y_e_i -= B_k_i U_e_k D_e_k C_k W_e", expected, B, U, D, C, W)
    expected = 2.0 * Y0 - expected
    tY.MoveFromGPU()
    assert rel_err(tY.data, expected) <= TOL


def test_dense_operator_applied_to_slices(at, engine, checker):
    """The entries' vectors and the results are slices of larger tensors (a slice starts at a whole number of rows,
    so the 16-byte loads of the entries' vectors stay aligned)."""
    rng = np.random.default_rng(5)
    B = rng.uniform(-1, 1, (16, 24))
    for entries in (50, 51):
        X = rng.uniform(-1, 1, (3, entries, 24))
        A0 = rng.uniform(-1, 1, (2, entries, 16))
        tX, tA, tB = to_tensor(at, X), to_tensor(at, A0), to_tensor(at, B)
        tA.MoveToGPU()
        engine("A_e_i = B_i_j X_e_j", at.SliceTensor(tA, 1), tB, at.SliceTensor(tX, 1))
        assert "matrix cores" in engine.GetLastImplementation()
        tA.MoveFromGPU()
        expected = np.zeros((entries, 16))
        checker.contract("A_e_i = B_i_j X_e_j", expected, B, np.ascontiguousarray(X[1]))
        assert rel_err(tA.data[1], expected) <= TOL and np.array_equal(tA.data[0], A0[0])


@pytest.mark.parametrize("m", [1, 2, 3])
def test_batched_matrices_at_odd_offsets(at, engine, checker, m):
    # slices whose first entry is 8 but not 16 bytes into the allocation, and a caller's device buffer likewise
    E = 5
    rng = np.random.default_rng(40 + m)
    J = np.eye(m) + 0.1 * rng.uniform(-1, 1, (3, E, m, m))
    tJ, tI, tD = to_tensor(at, J), at.Tensor(*J.shape), at.Tensor(3, E)
    for k in range(3):
        engine.BatchMatrixInvDet(at.SliceTensor(tI, k), at.SliceTensor(tD, k), at.SliceTensor(tJ, k))
    tI.MoveFromGPU()
    tD.MoveFromGPU()
    ri, rd = checker.batch_matrix_inv_det(J)
    assert np.array_equal(tI.data, ri) and np.array_equal(tD.data, rd)
    # a caller's device buffer one double into an allocation
    pool = at.Tensor(2 * J[0].size + 8)
    pool.MoveToGPU()
    host = np.ascontiguousarray(J[1])
    ext = at.Tensor(*host.shape, hdata=host, ddata=pool.GetDeviceData() + 8, ongpu=False)
    ext.MoveToGPU()
    inv, det = at.Tensor(*host.shape), at.Tensor(E)
    engine.BatchMatrixInvDet(inv, det, ext)
    inv.MoveFromGPU()
    det.MoveFromGPU()
    assert np.array_equal(inv.data, ri[1]) and np.array_equal(det.data, rd[1])


def test_operator_kernels_on_buffers_that_are_only_8_byte_aligned(at, engine, checker):
    # the operator schedule moves the entries' vectors with 16-byte instructions; a caller's device buffer one double
    # into an allocation must work like any other
    E, n = 300, 20
    rng = np.random.default_rng(77)
    B, X = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (E, n))
    pool = at.Tensor(2 * X.size + 16)
    pool.MoveToGPU()
    base = pool.GetDeviceData()
    hx, ha = X.copy(), np.zeros((E, n))
    tX = at.Tensor(E, n, hdata=hx, ddata=base + 8, ongpu=False)
    tA = at.Tensor(E, n, hdata=ha, ddata=base + 8 * (X.size + 3), ongpu=False)
    tX.MoveToGPU()
    engine("A_e_i = B_i_j X_e_j", tA, to_tensor(at, B), tX)
    assert "matrix cores" in engine.GetLastImplementation()
    tA.MoveFromGPU()
    expected = np.zeros((E, n))
    checker.contract("A_e_i = B_i_j X_e_j", expected, B, X)
    assert rel_err(ha, expected) <= 1e-12


@pytest.mark.parametrize("kernel,shapes,matrix_cores", [
    ("A_e_i_k = B_i_j X_e_j_k", [(64, 64), (333, 64, 3)], True),            # 999 entries (e, k): ragged last trip
    ("A_e_i_k += B_i_j X_e_j_k", [(16, 16), (1000, 16, 3)], True),
    ("A_e_i_k -= B_j_i X_e_j_k", [(33, 20), (77, 33, 2)], True),            # operator stored transposed, padded to 32 x 36
    ("A_e_q_i_k = B_i_j X_e_q_j_k", [(30, 17), (50, 4, 17, 5)], True),      # two leading indices, five components
    ("A_e_i_k_l = B_i_j X_e_j_k_l", [(24, 24), (101, 24, 2, 3)], True),     # two component indices
    ("V_e_q_c = B_q_i X_e_i_c", [(27, 27), (1001, 27, 3)], True),           # the components of an entry together, results through LDS
    ("V_e_q_c -= B_i_q X_e_i_c", [(16, 20), (517, 16, 2)], True),           # operator stored transposed, two components
    ("V_e_q_c = B_q_i X_e_i_c", [(125, 64), (203, 64, 3)], True),           # too large for LDS: two blocks of rows, components together
    ("V_e_q_c += B_q_i X_e_i_c", [(216, 125), (301, 125, 2)], True),        # blocks of rows, entries (entry, component)
    ("A_e_i_k = B_i_j X_e_j_k", [(8, 8), (1000, 8, 3)], False),             # small operator: the generic schedule
    ("A_e_i_k = B_i_j X_e_j_k W_e", [(32, 32), (100, 32, 3), (100,)], False),  # with a factor: the generic schedule
])
def test_dense_operator_with_trailing_components(at, engine, checker, kernel, shapes, matrix_cores):
    """The vectors and the results carry component indices behind the operator's ("A_e_i_k = B_i_j X_e_j_k", a vector
    field interpolated component by component): entries (e, k) with their elements a stride apart."""
    rng = np.random.default_rng(shapes[0][0] + shapes[1][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert ("operator schedule on the FP64 matrix cores" in src and "components per vector element" in src) == matrix_cores
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL
    # integer data: exact whatever the order of the sums
    ins = [rng.integers(-3, 4, s).astype(np.float64) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel.replace("+=", "=").replace("-=", "="), np.zeros_like(out0), *ins)
    assert np.array_equal(got, expected)


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i = B_i_j X_e_j", [(27, 3), (1000, 3)]),                # 27 results per lane: written out through an LDS tile
    ("A_e_i = B_i_j X_e_j", [(20, 5), (777, 5)]),                 # even run, last workgroup partly filled
    ("A_e_i_k = B_i_k_j X_e_j", [(5, 3, 3), (333, 3)]),           # the run spans two output dimensions
    ("A_e_i = X_e_j B_j_i", [(2, 9), (130, 2)]),
])
def test_long_output_runs_leave_through_an_lds_tile(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(shapes[1][0])
    if kernel.startswith("A_e_i = X"):
        shapes = [shapes[1], shapes[0]]
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "LDS tiles -> device memory" in engine.GetLastImplementation()
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e_i = B_e_i_j C_e_j", [(300, 21, 21), (300, 21)]),        # rows of 21: products into LDS, then row sums (from 25 on: matrix cores)
    ("A_e_i += B_e_i_j C_e_j", [(77, 9, 25), (77, 25)]),
    ("A_e_i -= C_e_j B_e_i_j", [(50, 33), (50, 12, 33)]),
    ("A_e_i = B_e_i_j_k C_e_j_k", [(40, 6, 3, 7), (40, 3, 7)]),   # two contraction indices, 21 terms
    ("A_e_i = B_e_i_j C_j", [(200, 27, 27), (27,)]),              # the vector shared by all entries
])
def test_element_matrix_times_vector_with_odd_rows(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "steps of:" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes,steps", [
    ("A_e = B_e_i", [(3001, 9)], True),                                   # row sums
    ("A_e += B_e_i C_e_i", [(2000, 27), (2000, 27)], True),               # dot products of short rows
    ("A_e -= B_i C_e_i", [(20,), (1234, 20)], True),                      # a weight vector shared by the entries
    ("A_e = B_e_i C_i D_e_i", [(500, 45), (45,), (500, 45)], True),       # three factors along the row
    ("A_e = B_e_i_j C_e_i_j", [(700, 3, 5), (700, 3, 5)], True),          # two contraction indices, rows of 15
    ("A_e_k = B_e_k_i C_e_i", [(600, 2, 27), (600, 27)], True),           # two sums per entry
    ("A_e_j = B_e_i_j C_e_i", [(700, 27, 2), (700, 27)], True),           # a vector applied from the left: sums down the columns
    ("A_e_j -= B_e_i_j", [(500, 64, 3)], True),                           # column sums
    ("A_e_j_k = B_e_i_j_k C_e_i", [(300, 20, 2, 2), (300, 20)], True),    # four columns numbered by two indices
    ("A_e_j = B_e_i_j C_i", [(500, 64, 2), (64,)], False),                # a vector that all entries share: as written
    ("A_e_j = B_e_i_j C_e_i", [(500, 12, 2), (500, 12)], False),          # few rows: as written
    ("A_e = B_e_i", [(5000, 5)], False),                                  # short rows and powers of two stay as they are
    ("A_e = B_e_i C_e_i", [(5000, 16), (5000, 16)], False),
    ("A_e = B_e_i_j C_i D_j", [(900, 7, 9), (7,), (9,)], False),          # factors along part of a row
])
def test_short_sums_per_entry_go_through_an_lds_tile(at, engine, checker, kernel, shapes, steps):
    # the products with the lanes along the operand as it lies in memory, into a tile in LDS, then a lane per sum
    rng = np.random.default_rng(shapes[0][0])
    ins = [rng.integers(-3, 4, s).astype(np.float64) for s in shapes]
    out0 = rng.integers(-3, 4, output_shape(kernel, shapes)).astype(np.float64)
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert ("steps of:" in engine.GetLastImplementation()) == steps
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("A_e = B_e_j C_e_i", [(3000, 32), (3000, 27)]),                         # both operands summed first, then one product
    ("A_e_l += B_i_l C_e_j_k", [(20, 10), (501, 64, 9)]),                    # the element tensor summed first
    ("A_e_i_j -= B_e_k C_e_i_j_l", [(333, 27), (333, 12, 20, 9)]),
    ("A_e_k = B_k_i C_e_j_k", [(12, 32), (2177, 64, 12)]),
])
def test_operands_that_carry_a_contraction_index_alone_are_summed_first(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(shapes[0][0])
    ins = [rng.integers(-3, 4, s).astype(np.float64) for s in shapes]
    out0 = rng.integers(-3, 4, output_shape(kernel, shapes)).astype(np.float64)
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "steps of:" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= 4 * TOL            # another order of additions than the oracle's


@pytest.mark.parametrize("n,m,op", [(5000, 8, "="), (3001, 4, "+="), (2500, 7, "-="), (2100, 11, "=")])
def test_small_gram_matrix_over_the_batch(at, engine, checker, n, m, op):
    # "A_i_j = B_e_i C_e_j": a contraction over the long index with m x m outputs that are products of two short loads;
    # up to 8 x 8 a lane owns whole slices (m + m loads, m x m accumulators), beyond that the matrix cores take over
    kernel = "A_i_j %s B_e_i C_e_j" % op
    rng = np.random.default_rng(n + m)
    B, C = rng.uniform(-1, 1, (n, m)), rng.uniform(-1, 1, (n, m))
    out0 = rng.uniform(-1, 1, (m, m))
    got, expected = run_single(at, engine, checker, kernel, out0, B, C)
    src = engine.GetLastImplementation()
    assert ("reduction schedule" in src and "a lane owns whole slices" in src) if m <= 8 else ("Gram schedule" in src)
    if op == "-=":
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL
    again, _ = run_single(at, engine, checker, kernel, out0, B, C)
    assert np.array_equal(got, again)                   # fixed order of additions: reproducible


@pytest.mark.parametrize("kernel,shapes", [
    ("A_i_j = B_e_i C_e_j", [(40000, 64), (40000, 64)]),                              # 16 blocks per wavefront
    ("A_j_i -= B_e_q_i C_e_q_j W_e_q", [(1001, 3, 40), (1001, 3, 50), (1001, 3)]),      # ragged everywhere, transposed, weighted
    ("A_i_j_k += C_n_j_k B_n_i", [(2300, 5, 7), (2300, 12)]),                           # operands the other way round: 35 x 12
    ("A_i_j = B_e_i C_e_j", [(2049, 16), (2049, 16)]),                                 # one more row than a multiple of four
])
def test_many_outputs_summed_over_the_batch(at, engine, checker, kernel, shapes):
    # more outputs than the reduction schedule takes: 16 x 16 blocks on the FP64 matrix cores, four rows of the range per
    # instruction, partial sums of the workgroups added by a second kernel in a fixed order
    rng = np.random.default_rng(shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    assert "Gram schedule on the FP64 matrix cores" in engine.GetLastImplementation()
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= 4 * TOL            # sums of 10^3 - 10^5 terms in another order than the oracle's
    again, _ = run_single(at, engine, checker, kernel, out0, *ins)
    assert np.array_equal(got, again)                   # reproducible


@pytest.mark.parametrize("kernel,shapes,expect", [
    ("S_i_j = A_e_i_j", [(3001, 32, 32)], "256 outputs per workgroup, a lane each"),            # the sum of element matrices
    ("S_i -= A_e_i B_e", [(2500, 5000), (2500,)], "256 outputs per workgroup, a lane each"),
    ("S_j_i += A_e_f_i_j B_e_f", [(700, 3, 9, 33), (700, 3)], "256 outputs per workgroup, a lane each"),   # 297 outputs, transposed, two summed indices
    ("S_i_j = A_e_i_j", [(4001, 12, 12)], "output entries on adjacent lanes"),                  # up to 256: every workgroup has them all
    ("S_i += A_i_e B_e", [(300, 5003), (5003,)], "four outputs per workgroup"),                  # summed index fastest: by rows
])
def test_sums_over_a_long_index_with_many_outputs(at, engine, checker, kernel, shapes, expect):
    rng = np.random.default_rng(shapes[0][0])
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert "reduction schedule" in src and expect in src
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= 4 * TOL            # sums of thousands of terms in another order than the oracle's
    again, _ = run_single(at, engine, checker, kernel, out0, *ins)
    assert np.array_equal(got, again)                   # fixed order of additions: reproducible


@pytest.mark.parametrize("kernel,shapes,expect", [
    # more than 128 outputs whose terms do not stream one operand once: every value of B goes into 16 outputs
    ("A_i_j += B_i_e C_j", [(12, 30011), (16,)], "four outputs per workgroup"),
    ("A_j_e = B_i_j C_e", [(50021, 9), (20,)], "output entries on adjacent lanes"),
    # more rows than one finishing workgroup has lanes, summed index fastest: by rows, a finishing workgroup per 256
    ("A_e -= B_i C_e_i", [(8192,), (2048, 8192)], "four outputs per workgroup"),
    ("S_i = A_i_e", [(1500, 9000)], "four outputs per workgroup"),
    # outputs and summed indices interleaved in the big operand, numbered in its memory order
    ("A_i_k = B_j_k_l C_e D_k_j_e_i", [(6, 9, 5), (700,), (9, 6, 700, 5)], "output entries on adjacent lanes"),
    ("A_i_j = B_k_i_e C_j_e_k", [(50, 27, 300), (8, 300, 50)], "four outputs per workgroup"),
    ("A_k_j_i += B_j_e_k C_i_j D_e_i", [(7, 9000, 12), (20, 7), (9000, 20)], "256 outputs per workgroup, a lane each"),
])
def test_long_contractions_of_any_layout_are_shared_out_over_workgroups(at, engine, checker, kernel, shapes, expect):
    # what no other schedule takes and the generic plan would leave to few lanes with hundreds of terms each
    rng = np.random.default_rng(shapes[0][0])
    ins = [rng.integers(-3, 4, s).astype(np.float64) for s in shapes]
    out0 = rng.integers(-3, 4, output_shape(kernel, shapes)).astype(np.float64)
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert "reduction schedule" in src and expect in src
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert np.array_equal(got, expected)               # small integers: exact in any order
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= 4 * TOL
    again, _ = run_single(at, engine, checker, kernel, out0, *ins)
    assert np.array_equal(got, again)                   # fixed order of additions: reproducible


@pytest.mark.parametrize("kernel,shapes,expect", [
    ("A_i_e = B_i_e C_i_e", [(16, 5000), (16, 5000)], "lanes(i)=16"),
    ("A_i_j_e -= B_i_k_e C_k_j_e", [(3, 3, 4099), (3, 3, 4099)], "lanes()=1 tile(i,j)=9"),          # ragged last workgroup
    ("A_i_e += B_i_k C_k_e W_e", [(5, 7), (7, 6001), (6001,)], "entry fastest"),
    ("A_e = B_e C_e", [(70001,), (70001,)], "256 per workgroup of 256 lanes, numbered with the entry fastest"),
])
def test_tensors_with_the_batch_index_last(at, engine, checker, kernel, shapes, expect):
    # structure-of-arrays layouts: the work items are numbered with the entry fastest, so that the lanes of a wavefront
    # read consecutive entries
    rng = np.random.default_rng(len(kernel))
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert "numbered with the entry fastest" in src and expect in src
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL


def test_repeated_captures_follow_changes_of_tensors_and_marks(at, engine, checker):
    # a repeated call with the same tensors reuses the previous binding; any change of a tensor, a buffer or a mark
    # must be seen: other tensors of the same shapes, a transient mark set and cleared, a slice of another parent
    rng = np.random.default_rng(77)
    E = 300
    B = rng.uniform(-1, 1, (5, 4))
    X1, X2 = rng.uniform(-1, 1, (E, 4)), rng.uniform(-1, 1, (E, 4))
    tB, tX1, tX2 = to_tensor(at, B), to_tensor(at, X1), to_tensor(at, X2)
    tU, tY1, tY2 = at.Tensor(E, 5), at.Tensor(E, 4), at.Tensor(E, 4)

    def run(tX, tY):
        engine.BeginMultiKernelLaunch()
        engine("U_e_q = B_q_i X_e_i", tU, tB, tX)
        engine("Y_e_i = B_q_i U_e_q", tY, tB, tU)
        engine.EndMultiKernelLaunch()
        tY.MoveFromGPU()
        return tY.data.copy()

    ref1, ref2 = (X1 @ B.T) @ B, (X2 @ B.T) @ B
    for _ in range(3):
        assert rel_err(run(tX1, tY1), ref1) <= TOL
    assert rel_err(run(tX2, tY1), ref2) <= TOL                 # another input
    assert rel_err(run(tX2, tY2), ref2) <= TOL                 # another output
    tU.SetTransient(True)                                      # U need not reach device memory any more
    tU.MoveToGPU()
    assert rel_err(run(tX1, tY1), ref1) <= TOL
    tU.SetTransient(False)
    assert rel_err(run(tX1, tY2), ref1) <= TOL
    tU.MoveFromGPU()
    assert rel_err(tU.data, X1 @ B.T) <= TOL                   # stored again
    # slices of two parents at the same place in the call
    P1, P2 = rng.uniform(-1, 1, (2, E, 4)), rng.uniform(-1, 1, (2, E, 4))
    tP1, tP2 = to_tensor(at, P1), to_tensor(at, P2)
    for parent, values in ((tP1, P1), (tP2, P2), (tP1, P1)):
        for k in (0, 1):
            assert rel_err(run(at.SliceTensor(parent, k), tY1), (values[k] @ B.T) @ B) <= TOL
    # single kernels: the same string on other tensors, then with the output as "+="
    for tX, X in ((tX1, X1), (tX2, X2), (tX1, X1)):
        engine("U_e_q = B_q_i X_e_i", tU, tB, tX)
        tU.MoveFromGPU()
        assert rel_err(tU.data, X @ B.T) <= TOL


def test_gram_matrix_of_one_tensor_and_of_slices(at, engine, checker):
    rng = np.random.default_rng(5)
    B = rng.uniform(-1, 1, (7001, 20))
    tB, tA = to_tensor(at, B), at.Tensor(20, 20)
    engine("A_i_j = B_e_i B_e_j", tA, tB, tB)                  # the same tensor on both sides
    tA.MoveFromGPU()
    assert "Gram schedule" in engine.GetLastImplementation() and rel_err(tA.data, B.T @ B) <= 4 * TOL
    big = rng.uniform(-1, 1, (2, 7001, 20))
    tbig = to_tensor(at, big)
    engine("A_i_j += B_e_i C_e_j", tA, at.SliceTensor(tbig, 1), at.SliceTensor(tbig, 0))   # views at an offset
    tA.MoveFromGPU()
    assert "Gram schedule" in engine.GetLastImplementation() and rel_err(tA.data, B.T @ B + big[1].T @ big[0]) <= 4 * TOL


@pytest.mark.parametrize("kernel,shapes", [
    ("J_e_q_n_m = G_q_i_n X_e_i_m", [(27, 27, 3), (501, 27, 3)]),                  # Jacobians: row indices q, n around the column index
    ("A_e_i1_i2 += B_i1_j1_i2_j2 X_e_j1_j2", [(6, 4, 5, 7), (1003, 4, 7)]),       # rows and columns interleaved
    ("A_e_i1_i2 -= B_j2_i2_j1_i1 X_e_j1_j2 W_e", [(7, 5, 4, 6), (777, 4, 7), (777,)]),   # every dimension the other way round
    ("G_e_d_q = D_q_i_d X_e_i", [(70, 64, 3), (1001, 64)]),                        # too large for LDS as well: blocks of rows
    ("J_e_q_m_n = X_e_i_m G_q_i_n", [(501, 27, 3), (27, 27, 3)]),                  # the component m between the row indices
    ("J_e_m_q_n += G_q_n_i X_e_i_m", [(13, 2, 10), (333, 10, 3)]),                 # ... in front of them, few rows
    ("J_e_q_m_n = X_e_i_m G_q_i_n", [(301, 64, 3), (64, 64, 3)]),                  # ... of an operator applied in blocks of rows
    # (its blocks of 128 rows do not fit the registers when the operator's values are kept across trips: compiled again without)
    ("O_e_i0_m0_i1_i2 += I0_e_j0_j1_m0 I1_j1_i0_i2_j0_i1", [(1368, 26, 2, 2), (2, 37, 3, 26, 10)]),
    ("J_e_q_m_k_n -= G_n_q_i X_e_i_m_k", [(3, 9, 10), (205, 10, 2, 2)]),           # two components, both between
])
def test_dense_operator_with_dimensions_in_any_order(at, engine, checker, kernel, shapes):
    rng = np.random.default_rng(len(kernel))
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    out0 = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, out0, *ins)
    src = engine.GetLastImplementation()
    assert "operator schedule on the FP64 matrix cores" in src and ("dimensions in another order" in src or "_m" in kernel)
    if "-=" in kernel:
        expected = 2.0 * out0 - expected
    assert rel_err(got, expected) <= TOL
