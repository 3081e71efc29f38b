"""Single kernels that the HIP policy evaluates as a chain of smaller contractions (partial results in LDS) must give
what the reference's interpreter gives for the kernel as written (exec/CPUInterpretedExecutor.cpp:59-121), for every
assignment operator, binding mode and index layout.  Through the C ABI, against the oracle."""
import numpy as np
import pytest

from gpu_helpers import output_shape, rel_err, run_single, to_tensor

pytestmark = pytest.mark.gpu
TOL = 1e-12


def is_reordered(engine):
    return "_F1" in engine.GetLastImplementation()


# kernel, input shapes; every one of them is large enough and gains enough for the generator to reorder it
REORDERED = [
    # p=2 mass assembly, config 3 of the baseline at a ragged element count
    ("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s", [(4, 3)] * 6 + [(37, 4, 4, 4)]),
    # the element index is not the first dimension of the output or of the streamed input
    ("M_i_j_e_k_l = B_q_i B_q_k B_r_j B_r_l W_q_e_r", [(6, 5)] * 4 + [(6, 50, 6)]),
    # three different tables, an input that has no contraction index at all (pointwise factor C_e)
    ("Y_e_a_b_c = P_a_i Q_b_j R_c_k X_e_i_j_k C_e", [(7, 6), (5, 6), (4, 6), (21, 6, 6, 6), (21,)]),
    # two contraction indices leave together (n and m only meet in F and G)
    ("Z_e_i_j = F_i_n_m G_n_m_p H_p_j_q X_e_q", [(9, 4, 3), (4, 3, 8), (8, 9, 7), (19, 7)]),
    # a contraction index that a single operand carries alone (T_e_i_j = sum_k A_e_i_j_k, then the rest)
    ("Y_e_i = A_e_i_j_k B_j_l C_l_m D_m_i", [(11, 12, 9, 8), (9, 10), (10, 9), (9, 12)]),
]


@pytest.mark.parametrize("op", ["=", "+=", "-="])
@pytest.mark.parametrize("kernel,shapes", REORDERED)
def test_reordered_kernel_matches_the_kernel_as_written(at, engine, checker, kernel, shapes, op):
    kernel = kernel.replace(" = ", " %s " % op)
    rng = np.random.default_rng(len(kernel) * 7 + len(op))
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    init = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, init, *ins)
    assert is_reordered(engine), engine.GetLastImplementation().splitlines()[1:6]
    if op == "-=":
        expected = init - (expected - init)  # the interpreter adds for "-=" (exec/CPUInterpretedExecutor.cpp:106)
    assert rel_err(got, expected) <= TOL


def test_reordered_kernel_is_exact_on_integer_data(at, engine, checker):
    kernel, shapes = REORDERED[0]
    ins = [np.arange(np.prod(s), dtype=np.float64).reshape(s) % 5 - 2.0 for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, np.zeros(output_shape(kernel, shapes)), *ins)
    assert is_reordered(engine)
    assert np.array_equal(got, expected)


def test_reordered_kernel_with_one_name_bound_to_two_tensors(at, engine, checker):
    # "B" names two different tensors: operands are taken by position (reference kernel/TensorEngine.cpp:290-336
    # passes the tensors of a call in order, whatever their names say)
    kernel = "M_e_i_j_k_l = B_q_i B_q_k B_r_j B_r_l W_e_q_r"
    rng = np.random.default_rng(5)
    tables = [rng.uniform(-1, 1, (6, 5)) for _ in range(4)]
    W = rng.uniform(0.5, 1.5, (40, 6, 6))
    got, expected = run_single(at, engine, checker, kernel, np.zeros((40, 5, 5, 5, 5)), *tables, W)
    assert is_reordered(engine)
    assert rel_err(got, expected) <= TOL
    assert rel_err(got, np.einsum("qi,qk,rj,rl,eqr->eijkl", *tables, W)) <= TOL


def test_reordered_kernel_writes_into_a_slice_and_reads_a_slice(at, engine, checker):
    rng = np.random.default_rng(6)
    B, W = rng.uniform(-1, 1, (6, 5)), rng.uniform(0.5, 1.5, (2, 30, 6, 6))
    tB, tW, M = to_tensor(at, B), to_tensor(at, W), at.Tensor(2, 30, 5, 5, 5, 5)
    M.Set(-1.0)
    M1, W1 = at.SliceTensor(M, 1), at.SliceTensor(tW, 1)
    engine("M_e_i_j_k_l = B_q_i B_q_k B_r_j B_r_l W_e_q_r", M1, tB, tB, tB, tB, W1)
    assert is_reordered(engine)
    M.MoveFromGPU()
    assert rel_err(M.data[1], np.einsum("qi,qk,rj,rl,eqr->eijkl", B, B, B, B, W[1])) <= TOL
    assert np.all(M.data[0] == -1.0)


def test_kernel_runs_as_written_when_no_partial_result_fits_in_lds(at, engine, checker):
    # both candidate partial results (8 x 800 doubles per batch entry) exceed 48 KB
    kernel = "Y_e_a_b = P_a_i Q_b_j X_e_i_j"
    shapes = [(8, 800), (8, 800), (10, 800, 800)]
    rng = np.random.default_rng(8)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, np.zeros((10, 8, 8)), *ins)
    assert not is_reordered(engine)
    assert rel_err(got, expected) <= TOL


def test_partial_results_that_do_not_fit_together_fall_back(at, engine, checker):
    # the cheapest order keeps two partial results of 17^3 doubles alive at once (79 KB) and no order with smaller
    # ones exists, so the kernel runs as written
    kernel = "Y_e_a_b_c = P_a_i Q_b_j R_c_k X_e_i_j_k"
    shapes = [(17, 17)] * 3 + [(18, 17, 17, 17)]
    rng = np.random.default_rng(9)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, np.zeros((18, 17, 17, 17)), *ins)
    assert not is_reordered(engine)
    assert rel_err(got, expected) <= TOL
    # one size down both fit (16^3 doubles each, 64 KB together) and the chain is used
    shapes = [(16, 16)] * 3 + [(17, 16, 16, 16)]
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    got, expected = run_single(at, engine, checker, kernel, np.zeros((17, 16, 16, 16)), *ins)
    assert is_reordered(engine)
    assert rel_err(got, expected) <= TOL


def random_multi_operand_kernel(rng):
    letters = list("abcdfghijklmnopqrstuvwxyz")
    n_out, n_con = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    names = list(rng.choice(letters, size=n_out + n_con, replace=False))
    out_idx, con_idx = names[:n_out], names[n_out:]
    extent = {n: int(rng.integers(1, 6)) for n in names}
    extent[out_idx[0]] = int(rng.integers(6, 40))              # the batch index
    n_in = int(rng.integers(3, 6))
    ins = []
    for v in range(n_in):
        k = int(rng.integers(1, min(4, len(names)) + 1))
        ins.append(list(rng.choice(names, size=k, replace=False)))
    for c in con_idx:
        if not any(c in i for i in ins):
            ins[int(rng.integers(0, n_in))].append(c)
    op = str(rng.choice(["=", "=", "+=", "-="]))
    kernel = "O_" + "_".join(out_idx) + " " + op + " " + " ".join("I%d_%s" % (v, "_".join(i)) for v, i in enumerate(ins))
    return kernel, tuple(extent[n] for n in out_idx), [tuple(extent[n] for n in i) for i in ins], op


@pytest.mark.parametrize("seed", range(60))
def test_random_kernels_reordered_whenever_possible(at, engine, checker, monkeypatch, seed):
    # the size and gain thresholds are switched off, so every kernel with a cheaper chain of steps takes that path:
    # odd index patterns (inputs without the batch index, indices shared by all operands, broadcast output indices,
    # several indices leaving in one step) go through the ordering search and the LDS-only partial results
    monkeypatch.setenv("ACRO_HIP_FACTORISE", "2")
    rng = np.random.default_rng(9000 + seed)
    kernel, out_shape, shapes, op = random_multi_operand_kernel(rng)
    print(kernel, out_shape, shapes, flush=True)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    init = rng.uniform(-1, 1, out_shape)
    out = to_tensor(at, init)
    engine(kernel, out, *[to_tensor(at, a) for a in ins])
    out.MoveFromGPU()
    expected = init.copy()
    checker.contract(kernel.replace("-=", "+="), expected, *ins)
    if op == "-=":
        expected = init - (expected - init)
    assert rel_err(out.data, expected) <= TOL


@pytest.mark.parametrize("transient", [False, True])
def test_kernel_inside_a_multi_kernel_launch_is_reordered_too(at, engine, checker, transient):
    # assemble the element matrices and apply them in one launch: the 7-operand assembly kernel runs as three steps,
    # its result M feeds the next kernel from LDS (and is not stored at all when marked transient)
    rng = np.random.default_rng(12)
    E = 29
    B, W, X = rng.uniform(-1, 1, (4, 3)), rng.uniform(0.5, 1.5, (E, 4, 4, 4)), rng.uniform(-1, 1, (E, 3, 3, 3))
    tB, tW, tX = to_tensor(at, B), to_tensor(at, W), to_tensor(at, X)
    M, Y = at.Tensor(E, 3, 3, 3, 3, 3, 3), at.Tensor(E, 3, 3, 3)
    M.SetTransient(transient)
    engine.BeginMultiKernelLaunch()
    engine("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s", M, tB, tB, tB, tB, tB, tB, tW)
    engine("Y_e_i_j_k = M_e_i_j_k_l_m_n X_e_l_m_n", Y, M, tX)
    engine.EndMultiKernelLaunch()
    src = engine.GetLastImplementation()
    assert "_F1" in src and "_F2" in src and src.count("__global__") == 1
    assert ("M->lds\n" in src) == transient
    expM = np.zeros((E, 3, 3, 3, 3, 3, 3))
    checker.contract("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s", expM, B, B, B, B, B, B, W)
    expY = np.zeros((E, 3, 3, 3))
    checker.contract("Y_e_i_j_k = M_e_i_j_k_l_m_n X_e_l_m_n", expY, expM, X)
    Y.MoveFromGPU()
    assert rel_err(Y.data, expY) <= TOL
    if not transient:
        M.MoveFromGPU()
        assert rel_err(M.data, expM) <= TOL


# Kernels far above the machine balance (long contractions that every operand carries, many outputs): the contraction
# runs as counted loops around a register tile, tile operands from scalar registers where they do not depend on lanes.
LOOPED_TILE = [
    ("A_e_i_j_p_q = I0_p_k I1_i_k I2_q_k I3_e_k I4_j_k", [(7, 50), (4, 50), (4, 50), (33, 50), (8, 50)]),
    ("A_e_i_j_p_q = I0_k_l_m_j I1_p_k_l_m I2_e_k_l_m I3_k_l_m_q I4_i_k_l_m", [(4, 7, 6, 6), (6, 4, 7, 6), (18, 4, 7, 6), (4, 7, 6, 3), (5, 4, 7, 6)]),
    ("A_i_e_j_p_q = I0_q_k_l I1_e_k_l I2_p_k_l I3_j_k I4_i_k_l", [(2, 8, 7), (8, 8, 7), (8, 8, 7), (3, 8), (4, 8, 7)]),
    ("A_e_i_j_p_q = I0_j_k I1_i_k I2_e_k_q I3_p_k", [(3, 76), (6, 76), (16, 76, 6), (4, 76)]),
    ("A_e_i_j_p_q = I0_e_k_l_q I1_q_k_l I2_k_l_i I3_k_l_j I4_p_k_l", [(26, 6, 6, 7), (7, 6, 6), (6, 6, 7), (6, 6, 8), (6, 6, 6)]),
    ("A_e_i_j_p_q = I0_l_q I1_p_k_l I2_e_k_l_q I3_k_l_j I4_i_l", [(7, 8), (4, 6, 7), (7, 6, 7, 8), (6, 7, 4), (3, 7)]),
]


@pytest.mark.parametrize("op", ["=", "+=", "-="])
@pytest.mark.parametrize("kernel,shapes", LOOPED_TILE)
def test_compute_bound_kernel_loops_around_a_register_tile(at, engine, checker, kernel, shapes, op):
    kernel = kernel.replace(" = ", " %s " % op)
    rng = np.random.default_rng(len(kernel) * 11 + len(op))
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    init = rng.uniform(-1, 1, output_shape(kernel, shapes))
    got, expected = run_single(at, engine, checker, kernel, init, *ins)
    assert "around a register tile" in engine.GetLastImplementation()
    if op == "-=":
        expected = init - (expected - init)
    assert rel_err(got, expected) <= TOL


@pytest.mark.parametrize("transient", [False, True])
def test_stiffness_assembly_step_loops_around_a_register_tile(at, engine, checker, transient):
    # 3D stiffness assembly (reference unittest/kernel/test_TensorEngine.cpp:437-496): the k3 sum first, then 225 terms
    # per output around a 5 x 5 tile of outputs with one table in scalar registers; followed here by a pointwise kernel
    # that reads the result (from device memory: 15 625 outputs per element are no LDS tile)
    k = "S_e_i1_i2_i3_j1_j2_j3 = B1_i1_j1_k1_m_n B2_i2_j2_k2_m_n B3_i3_j3_k3_m_n D_e_k1_k2_k3_m_n"
    rng = np.random.default_rng(5)
    E = 3
    tables = [rng.integers(-2, 3, (5, 5, 5, 3, 3)).astype(np.float64) for _ in range(3)]
    D = rng.integers(-2, 3, (E, 5, 5, 5, 3, 3)).astype(np.float64)
    W = rng.integers(-2, 3, (E, 5, 5, 5, 5, 5, 5)).astype(np.float64)
    tS, tZ = at.Tensor(E, 5, 5, 5, 5, 5, 5), at.Tensor(E, 5, 5, 5, 5, 5, 5)
    tS.SetTransient(transient)
    tin = [to_tensor(at, a) for a in tables + [D]]
    tW = to_tensor(at, W)
    engine.BeginMultiKernelLaunch()
    engine(k, tS, *tin)
    engine("Z_e_i1_i2_i3_j1_j2_j3 = S_e_i1_i2_i3_j1_j2_j3 W_e_i1_i2_i3_j1_j2_j3", tZ, tS, tW)
    engine.EndMultiKernelLaunch()
    assert "around a register tile" in engine.GetLastImplementation()
    expected = np.zeros((E, 5, 5, 5, 5, 5, 5))
    checker.contract(k, expected, *tables, D)
    tZ.MoveFromGPU()
    assert np.array_equal(tZ.data, expected * W)          # small integers: exact
    if not transient:
        tS.MoveFromGPU()
        assert np.array_equal(tS.data, expected)
