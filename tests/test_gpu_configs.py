"""The five baseline configurations on the GPU: parity with the checker at sizes it finishes in seconds, the golden
fixtures written by the compiled reference, and size-independent properties at the full sizes."""
import os

import numpy as np
import pytest

from acrotensor_amd import workloads
from gpu_helpers import rel_err, to_tensor

pytestmark = pytest.mark.gpu
TOL = 1e-12          # max |gpu - cpu| / max |cpu| per output tensor, fp64
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def run_workload(at, engine, wl, transient):
    print("workload:", wl.name, "transient" if transient else "stored", flush=True)
    tensors = workloads.bind_to_engine(wl, at, transient=transient)
    workloads.launch(wl, engine, tensors)
    return tensors


def fetch(tensors, name):
    tensors[name].MoveFromGPU()
    return tensors[name].data.copy()


@pytest.mark.parametrize("n", [1, 63, 4096, 100003])
def test_config1_batched_reduction(at, engine, checker, n):
    wl = workloads.config1(n=n)
    tensors = run_workload(at, engine, wl, False)
    expected = workloads.run_on_checker(wl, checker)["S"]
    assert rel_err(fetch(tensors, "S"), expected) <= TOL


def test_config1_integer_data_is_exact(at, engine):
    n = 50000
    A = (np.arange(n * 9) % 17).astype(np.float64).reshape(n, 3, 3)
    S = at.Tensor(3, 3)
    engine("S_i_j = A_n_i_j B_n", S, to_tensor(at, A), to_tensor(at, np.ones(n)))
    S.MoveFromGPU()
    assert np.array_equal(S.data, A.sum(axis=0))


@pytest.mark.parametrize("E,Q", [(1, 1), (3, 64), (100, 64)])
def test_config2_jacobian_inverse_determinant(at, engine, checker, E, Q):
    J = workloads.config2_inputs(E=E, Q=Q)
    tJ, Jinv, Jdet = to_tensor(at, J), at.Tensor(E, Q, 3, 3), at.Tensor(E, Q)
    engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
    ri, rd = checker.batch_matrix_inv_det(J)
    assert np.array_equal(fetch({"a": Jinv}, "a"), ri) and np.array_equal(fetch({"a": Jdet}, "a"), rd)


@pytest.mark.parametrize("E", [1, 7, 64])
def test_config3_mass_assembly(at, engine, checker, E):
    wl = workloads.config3(E=E)
    tensors = run_workload(at, engine, wl, False)
    expected = workloads.run_on_checker(wl, checker)["M"]
    assert rel_err(fetch(tensors, "M"), expected) <= TOL


@pytest.mark.parametrize("E", [1, 3, 8, 333, 1024])
@pytest.mark.parametrize("transient", [False, True])
def test_config4_mass_apply(at, engine, checker, E, transient):
    wl = workloads.config4(E=E)
    tensors = run_workload(at, engine, wl, transient)
    expected = workloads.run_on_checker(wl, checker)
    assert rel_err(fetch(tensors, "Y"), expected["Y"]) <= TOL
    if not transient:                                      # every intermediate is a valid tensor after the launch
        for name in wl.transient:
            assert rel_err(fetch(tensors, name), expected[name]) <= TOL, name


@pytest.mark.parametrize("E,Q,P", [(61, 3, 2), (45, 4, 3), (131, 5, 4), (26, 6, 5), (13, 7, 6), (7, 8, 7), (5, 9, 8), (3, 10, 9)])
@pytest.mark.parametrize("transient", [False, True])
def test_mass_apply_at_other_degrees(at, engine, checker, E, Q, P, transient):
    # the same 7-kernel chain at degrees 1 - 8: element counts that leave the last workgroup partly filled, every
    # intermediate stored (the batches that leave through LDS tiles) and transient (the prefetch rules)
    wl = workloads.config4(E=E, Q=Q, P=P)
    tensors = run_workload(at, engine, wl, transient)
    expected = workloads.run_on_checker(wl, checker)
    assert rel_err(fetch(tensors, "Y"), expected["Y"]) <= TOL
    if not transient:
        for name in wl.transient:
            assert rel_err(fetch(tensors, name), expected[name]) <= TOL, name


@pytest.mark.parametrize("E,Q,P", [(1, 5, 4), (5, 5, 4), (3, 10, 8), (23, 3, 2), (19, 4, 3), (7, 6, 5), (3, 7, 6)])
@pytest.mark.parametrize("transient", [False, True])
def test_config5_diffusion_apply(at, engine, checker, E, Q, P, transient):
    wl = workloads.config5(E=E, Q=Q, P=P)
    tensors = run_workload(at, engine, wl, transient)
    expected = workloads.run_on_checker(wl, checker)
    assert rel_err(fetch(tensors, "Y"), expected["Y"]) <= TOL
    if not transient:
        for name in ("U", "Z"):
            assert rel_err(fetch(tensors, name), expected[name]) <= TOL, name


def golden_workloads():
    return sorted(f for f in os.listdir(GOLDEN) if f.startswith("workload_")) if os.path.isdir(GOLDEN) else []


@pytest.mark.parametrize("fname", golden_workloads())
def test_golden_workloads_of_the_compiled_reference(at, engine, fname):
    g = np.load(os.path.join(GOLDEN, fname), allow_pickle=False)
    kwargs = {str(k): int(v) for k, v in zip(g["arg_names"], g["arg_values"])}
    wl = getattr(workloads, str(g["config"]))(**kwargs)
    tensors = run_workload(at, engine, wl, True)
    for o in wl.outputs:
        assert rel_err(fetch(tensors, o), g["out_" + o]) <= TOL


def test_golden_invdet_of_the_compiled_reference(at, engine):
    g = np.load(os.path.join(GOLDEN, "cfg2_invdet_64.npz"), allow_pickle=False)
    A = np.ascontiguousarray(g["A"])
    tA, Ainv, Adet = to_tensor(at, A), at.Tensor(*A.shape), at.Tensor(*A.shape[:-2])
    engine.BatchMatrixInvDet(Ainv, Adet, tA)
    Ainv.MoveFromGPU()
    Adet.MoveFromGPU()
    assert np.array_equal(Ainv.data, g["Ainv"]) and np.array_equal(Adet.data, g["det"])


# ----------------------------------------------------------------------------- full-size properties

def test_config4_full_size_properties(at, engine, checker):
    """E = 2^18: sampled elements against the checker, linearity in X, and the constant-X closed form."""
    E = 262144
    wl = workloads.config4(E=E)
    tensors = run_workload(at, engine, wl, True)
    Y = fetch(tensors, "Y")
    B, X, D = wl.arrays["B"], wl.arrays["X"], wl.arrays["D"]
    # (1) elements 0, 1, E/2, E-1 and a strided sample, recomputed by the checker from the same inputs
    sample = np.array(sorted(set([0, 1, E // 2, E - 1] + list(range(5, E, E // 61)))))
    sub = workloads.config4(E=len(sample))
    sub.arrays["B"][...] = B
    sub.arrays["X"][...] = X[sample]
    sub.arrays["D"][...] = D[sample]
    expected = workloads.run_on_checker(sub, checker)["Y"]
    assert rel_err(Y[sample], expected) <= TOL
    # (1b) every element against the chain evaluated with numpy (different summation order: 1e-12, not bit-exact)
    T = np.einsum("qi,eijk->eqjk", B, X)
    T = np.einsum("rj,eqjk->eqrk", B, T)
    T = np.einsum("sk,eqrk->eqrs", B, T) * D
    T = np.einsum("qi,eqrs->eirs", B, T)
    T = np.einsum("rj,eirs->eijs", B, T)
    T = np.einsum("sk,eijs->eijk", B, T)
    per_element = np.abs(Y - T).reshape(E, -1).max(axis=1)
    assert per_element.max() <= TOL * np.abs(T).max(), "first bad element %d" % int(per_element.argmax())
    # (2) linearity: apply(2 X) = 2 apply(X) exactly (scaling by 2 is exact in binary floating point)
    tensors["X"].data[...] = 2.0 * X
    tensors["X"].SwitchFromGPU()
    workloads.launch(wl, engine, tensors)
    assert np.array_equal(fetch(tensors, "Y"), 2.0 * Y)
    # (3) X == 1, D == 1: Y_ijk = sum_qrs B_qi B_rj B_sk (sum_l B_ql)(sum_m B_rm)(sum_n B_sn), the same in every element
    for name, val in (("X", 1.0), ("D", 1.0)):
        tensors[name].SwitchFromGPU()
        tensors[name].Set(val)
    workloads.launch(wl, engine, tensors)
    Y1 = fetch(tensors, "Y")
    v = B.T @ B.sum(axis=1)
    closed = np.einsum("i,j,k->ijk", v, v, v)
    assert rel_err(Y1[0], closed) <= TOL
    assert np.array_equal(Y1, np.broadcast_to(Y1[0], Y1.shape))


def numpy_diffusion(wl):
    B, G, X, D = (wl.arrays[n] for n in "BGXD")
    combos = ((G, B, B), (B, G, B), (B, B, G))
    U = np.stack([np.einsum("qi,rj,sk,eijk->eqrs", a, b, c, X, optimize=True) for a, b, c in combos])
    Z = np.einsum("eqrsmn,neqrs->meqrs", D, U)
    return sum(np.einsum("qi,rj,sk,eqrs->eijk", a, b, c, Z[m], optimize=True) for m, (a, b, c) in enumerate(combos))


def test_config5_every_element_against_numpy(at, engine):
    """p=7 diffusion apply on 4096 elements: every element against the operator evaluated with numpy."""
    wl = workloads.config5(E=4096)
    tensors = run_workload(at, engine, wl, True)
    Y = fetch(tensors, "Y")
    expected = numpy_diffusion(wl)
    per_element = np.abs(Y - expected).reshape(4096, -1).max(axis=1)
    assert per_element.max() <= TOL * np.abs(expected).max(), "first bad element %d" % int(per_element.argmax())
    # run to run reproducibility (no atomics, fixed summation order)
    workloads.launch(wl, engine, tensors)
    assert np.array_equal(fetch(tensors, "Y"), Y)


def test_config5_full_size_properties(at, engine, checker):
    """E = 65536 (D alone is 4.7 GB, more bytes than an int can count): sampled elements against the checker and
    exact linearity in X."""
    E = 65536
    wl = workloads.config5(E=E)
    tensors = run_workload(at, engine, wl, True)
    Y = fetch(tensors, "Y")
    sample = np.array([0, 1, E // 2, E - 1, 12345])
    sub = workloads.config5(E=len(sample))
    for name in ("B", "G"):
        sub.arrays[name][...] = wl.arrays[name]
    for name in ("X", "D"):
        sub.arrays[name][...] = wl.arrays[name][sample]
    expected = workloads.run_on_checker(sub, checker)["Y"]
    assert rel_err(Y[sample], expected) <= TOL
    tensors["X"].data[...] = 2.0 * wl.arrays["X"]
    tensors["X"].SwitchFromGPU()
    workloads.launch(wl, engine, tensors)
    assert np.array_equal(fetch(tensors, "Y"), 2.0 * Y)


def test_config2_full_size_properties(at, engine):
    """4 194 304 matrices: J (Jinv)^T = I and det(J) det(Jinv) = 1 everywhere."""
    J = workloads.config2_inputs()
    E, Q = J.shape[:2]
    tJ, Jinv, Jdet, Jdet2 = to_tensor(at, J), at.Tensor(E, Q, 3, 3), at.Tensor(E, Q), at.Tensor(E, Q)
    engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
    engine.BatchMatrixDet(Jdet2, Jinv)
    for t in (Jinv, Jdet, Jdet2):
        t.MoveFromGPU()
    prod = np.einsum("...ij,...kj->...ik", J, Jinv.data)
    assert np.abs(prod - np.eye(3)).max() < 1e-13
    assert np.abs(Jdet.data * Jdet2.data - 1.0).max() < 1e-13


def test_config1_full_size_closed_form(at, engine):
    wl = workloads.config1()
    tensors = run_workload(at, engine, wl, False)
    S = fetch(tensors, "S")
    expected = wl.arrays["A"].sum(axis=0, dtype=np.longdouble).astype(np.float64)
    assert rel_err(S, expected) <= TOL


@pytest.mark.parametrize("one_pass", [False, True])
def test_config1_repeated_launches_are_bit_identical_and_accumulate(at, engine, monkeypatch, one_pass):
    # the partial sums of the split contraction are added in a fixed order, by a second kernel or (experiment
    # switch) by whichever workgroup finishes last; neither the result nor the state left behind for the next launch
    # may depend on timing
    if one_pass:
        monkeypatch.setenv("ACRO_HIP_ONE_PASS", "1")
    wl = workloads.config1(n=1048576 - 8 * one_pass)
    tensors = run_workload(at, engine, wl, False)
    first = fetch(tensors, "S")
    k, out, ins = wl.kernels[0]
    for _ in range(50):
        engine(k, tensors[out], *[tensors[n] for n in ins])
    assert np.array_equal(fetch(tensors, "S"), first)
    tensors["S"].MoveToGPU()
    for _ in range(3):
        engine(k.replace(" = ", " += "), tensors[out], *[tensors[n] for n in ins])
    got = fetch(tensors, "S")
    assert rel_err(got, 4.0 * first) <= TOL
    # and a second shape on the same engine (its own scratch buffer and counter)
    n = 300007 + one_pass
    A = (np.arange(n * 9) % 13).astype(np.float64).reshape(n, 3, 3)
    S = at.Tensor(3, 3)
    tA, tB = to_tensor(at, A), to_tensor(at, np.ones(n))
    for _ in range(5):
        engine("S_i_j = A_n_i_j B_n", S, tA, tB)
    S.MoveFromGPU()
    assert np.array_equal(S.data, A.sum(axis=0))


def test_config3_full_size_symmetry_and_sample(at, engine, checker):
    E = 32768
    wl = workloads.config3(E=E)
    tensors = run_workload(at, engine, wl, False)
    M = fetch(tensors, "M")
    # the element mass matrix is symmetric: M[e,i,j,k,l,m,n] = M[e,l,m,n,i,j,k]
    Mt = M.transpose(0, 4, 5, 6, 1, 2, 3)
    assert np.abs(M - Mt).max() <= 1e-13 * np.abs(M).max()
    sample = np.array([0, 1, E // 2, E - 1])
    sub = workloads.config3(E=len(sample))
    sub.arrays["B"][...] = wl.arrays["B"]
    sub.arrays["W"][...] = wl.arrays["W"][sample]
    assert rel_err(M[sample], workloads.run_on_checker(sub, checker)["M"]) <= TOL


def test_node_vector_to_element_vector_and_back_full_size(at, engine):
    # FlatIndexedScatter / FlatIndexedSumGather on the mesh of the headline configuration (64^3 hexahedra of degree
    # 3: 16.8 M element entries, 7.2 M nodes); integer-valued data make every sum exact whatever the row length
    dofs, nodes = workloads.hex_mesh_dof_map(64, 64, 64, 3)
    M = at.IndexMapping(nodes, dofs.size)
    M.map[:] = dofs.ravel()
    Lv = (np.arange(nodes) % 97 - 48).astype(np.float64)
    L, Ev, back = to_tensor(at, Lv), at.Tensor(dofs.size), at.Tensor(nodes)
    engine.FlatIndexedScatter(Ev, L, M)
    Ev.MoveFromGPU()
    assert np.array_equal(Ev.data, Lv[dofs.ravel()])
    engine.FlatIndexedSumGather(back, Ev, M)
    back.MoveFromGPU()
    multiplicity = np.bincount(dofs.ravel(), minlength=nodes)
    assert multiplicity.min() == 1 and multiplicity.max() == 8
    assert np.array_equal(back.data, multiplicity * Lv)
