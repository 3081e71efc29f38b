"""A FlatIndexedScatter recorded inside a multi-kernel launch whose result is transient is not run: the kernels read
the source vector through the index map (node vector -> operator apply without the element vector ever existing).
Expected values: the checker's scatter followed by the checker's kernels."""
import numpy as np
import pytest

from acrotensor_amd import workloads
from gpu_helpers import rel_err, to_tensor

pytestmark = pytest.mark.gpu
TOL = 1e-12


def mesh(at, n, p):
    dofs, nodes = workloads.hex_mesh_dof_map(n, n, n, p)
    M = at.IndexMapping(nodes, dofs.size)
    M.map[:] = dofs.ravel()
    return dofs, nodes, M


@pytest.mark.parametrize("transient_x", [True, False])
@pytest.mark.parametrize("n", [3, 5])
def test_mass_apply_reads_the_node_vector_through_the_map(at, engine, checker, n, transient_x):
    dofs, nodes, M = mesh(at, n, 3)
    E = dofs.shape[0]
    wl = workloads.config4(E=E)
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    Lv = np.random.default_rng(n).uniform(-1, 1, nodes)
    L = to_tensor(at, Lv)
    tensors["X"].data[...] = -5.0
    tensors["X"].SetTransient(transient_x)
    engine.BeginMultiKernelLaunch()
    engine.FlatIndexedScatter(tensors["X"], L, M)
    for k, out, ins in wl.kernels:
        engine(k, tensors[out], *[tensors[i] for i in ins])
    engine.EndMultiKernelLaunch()
    src = engine.GetLastImplementation()
    assert ("X<-gathered" in src) == transient_x
    tensors["Y"].MoveFromGPU()
    arrays = {k: v.copy() for k, v in wl.arrays.items()}
    arrays["X"] = Lv[dofs.ravel()].reshape(arrays["X"].shape)
    wl.arrays.update(arrays)
    expected = workloads.run_on_checker(wl, checker)
    assert rel_err(tensors["Y"].data, expected["Y"]) <= TOL
    if not transient_x:                       # the element vector exists, as after a scatter on its own
        tensors["X"].MoveFromGPU()
        assert np.array_equal(tensors["X"].data, arrays["X"])


def test_single_kernel_counted_loops_and_lane_sharing_read_through_the_map(at, engine, checker):
    rng = np.random.default_rng(3)
    nodes, E, n = 500, 77, 40
    idx = rng.integers(0, nodes, E * n).astype(np.int32)
    M = at.IndexMapping(nodes, E * n)
    M.map[:] = idx
    Lv, Wv = rng.uniform(-1, 1, nodes), rng.uniform(-1, 1, (E, n))
    for kernel, oshape in (("A_e = X_e_n W_e_n", (E,)), ("A_e_n = X_e_n W_e_n", (E, n)), ("A_e_m = X_e_n B_m_n", (E, 700))):
        L, W = to_tensor(at, Lv), to_tensor(at, Wv)
        X, A = at.Tensor(E, n), at.Tensor(*oshape)
        X.SetTransient(True)
        second = W if "W_" in kernel else to_tensor(at, rng.uniform(-1, 1, (700, n)))
        engine.BeginMultiKernelLaunch()
        engine.FlatIndexedScatter(X, L, M)
        engine(kernel, A, X, second)
        engine.EndMultiKernelLaunch()
        assert "X<-gathered" in engine.GetLastImplementation(), kernel
        A.MoveFromGPU()
        expected = np.zeros(oshape)
        checker.contract(kernel, expected, Lv[idx].reshape(E, n), np.ascontiguousarray(second.data))
        assert rel_err(A.data, expected) <= TOL, kernel


def test_scatters_that_must_run(at, engine, checker):
    rng = np.random.default_rng(4)
    nodes, E, n = 300, 31, 8
    idx = rng.integers(0, nodes, E * n).astype(np.int32)
    M = at.IndexMapping(nodes, E * n)
    M.map[:] = idx
    Lv = rng.uniform(-1, 1, nodes)
    gathered = Lv[idx].reshape(E, n)
    # a kernel recorded before the scatter reads the old element vector; a kernel after it the new one
    L, X, A, B = to_tensor(at, Lv), to_tensor(at, np.full((E, n), 2.0)), at.Tensor(E, n), at.Tensor(E, n)
    X.SetTransient(True)
    engine.BeginMultiKernelLaunch()
    engine("A_e_n = X_e_n X_e_n", A, X, X)
    engine.FlatIndexedScatter(X, L, M)
    engine("B_e_n = X_e_n X_e_n", B, X, X)
    engine.EndMultiKernelLaunch()
    A.MoveFromGPU()
    B.MoveFromGPU()
    assert np.array_equal(A.data, np.full((E, n), 4.0)) and rel_err(B.data, gathered * gathered) <= TOL
    # the source vector is written by a kernel of the capture
    L2, S = at.Tensor(nodes), to_tensor(at, rng.uniform(-1, 1, nodes))
    X2, C = at.Tensor(E, n), at.Tensor(E, n)
    X2.SetTransient(True)
    engine.BeginMultiKernelLaunch()
    engine("L_i = S_i S_i", L2, S, S)
    engine.FlatIndexedScatter(X2, L2, M)
    engine("C_e_n = X_e_n X_e_n", C, X2, X2)
    engine.EndMultiKernelLaunch()
    C.MoveFromGPU()
    l2 = S.data * S.data
    assert rel_err(C.data, (l2[idx] ** 2).reshape(E, n)) <= TOL
    # nobody reads the result inside the capture: it exists afterwards
    X3 = at.Tensor(E, n)
    engine.BeginMultiKernelLaunch()
    engine.FlatIndexedScatter(X3, L, M)
    engine.EndMultiKernelLaunch()
    X3.MoveFromGPU()
    assert np.array_equal(X3.data, gathered)


def test_full_mesh_apply_through_the_map_equals_scatter_then_apply(at, engine):
    # 64^3 elements of degree 3 (the size bench.py measures): same arithmetic on the same values, so bit for bit
    dofs, nodes, M = mesh(at, 64, 3)
    wl = workloads.config4(E=dofs.shape[0])
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    L = to_tensor(at, workloads.counter_uniform(0xAC29, 0, (nodes,), -1.0, 1.0))

    def apply(through_map):
        tensors["X"].SetTransient(through_map)
        engine.BeginMultiKernelLaunch()
        engine.FlatIndexedScatter(tensors["X"], L, M)
        for k, out, ins in wl.kernels:
            engine(k, tensors[out], *[tensors[i] for i in ins])
        engine.EndMultiKernelLaunch()
        assert ("X<-gathered" in engine.GetLastImplementation()) == through_map
        tensors["Y"].MoveFromGPU()
        y = tensors["Y"].data.copy()
        tensors["Y"].MoveToGPU()
        tensors["Y"].Set(0.0)
        return y

    fused, separate = apply(True), apply(False)
    assert np.abs(separate).max() > 0.0 and np.array_equal(fused, separate)


def test_apply_through_the_map_replays_from_a_recorded_launch_sequence(at, engine, checker):
    dofs, nodes, M = mesh(at, 4, 3)
    wl = workloads.config4(E=dofs.shape[0])
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    tensors["X"].SetTransient(True)
    rng = np.random.default_rng(12)
    L = to_tensor(at, rng.uniform(-1, 1, nodes))

    def step():
        engine.BeginMultiKernelLaunch()
        engine.FlatIndexedScatter(tensors["X"], L, M)
        for k, out, ins in wl.kernels:
            engine(k, tensors[out], *[tensors[i] for i in ins])
        engine.EndMultiKernelLaunch()

    step()
    with at.recorded_launches() as recording:
        step()
    for _ in range(3):
        L.Mult(-0.5)                                      # eager work between the replays: a new node vector
        at.synchronize()
        recording.launch()
        tensors["Y"].MoveFromGPU()
        replayed = tensors["Y"].data.copy()
        tensors["Y"].MoveToGPU()
        tensors["Y"].Set(0.0)
        step()
        tensors["Y"].MoveFromGPU()
        assert np.abs(replayed).max() > 0.0 and np.array_equal(replayed, tensors["Y"].data)
        tensors["Y"].MoveToGPU()


def test_sum_gather_recorded_in_a_capture_runs_at_its_place(at, engine, checker):
    # node vector -> element vector -> mass apply -> node vector in ONE capture: the sum-gather is recorded like the
    # scatter and the kernels and takes effect after the kernels recorded before it
    dofs, nodes = workloads.hex_mesh_dof_map(3, 2, 2, 3)
    E = dofs.shape[0]
    for transient_x in (False, True):
        wl = workloads.config4(E=E)
        tensors = workloads.bind_to_engine(wl, at, transient=True)
        tensors["X"].SetTransient(transient_x)
        M = at.IndexMapping(nodes, dofs.size)
        M.map[:] = dofs.ravel()
        rng = np.random.default_rng(5)
        Lv = rng.uniform(-1, 1, nodes)
        L, Lout = to_tensor(at, Lv), at.Tensor(nodes)
        Lout.data[...] = -7.0
        engine.BeginMultiKernelLaunch()
        engine.FlatIndexedScatter(tensors["X"], L, M)
        for k, out, ins in wl.kernels:
            engine(k, tensors[out], *[tensors[n] for n in ins])
        engine.FlatIndexedSumGather(Lout, tensors["Y"], M)
        engine.EndMultiKernelLaunch()
        Lout.MoveFromGPU()
        wl.arrays["X"][...] = Lv[dofs]
        Y = workloads.run_on_checker(wl, checker)["Y"]
        expected = np.zeros(nodes)
        np.add.at(expected, dofs.ravel(), Y.ravel())
        assert rel_err(Lout.data, expected) <= 1e-12, transient_x
