"""Recorded launch sequences (hipGraph) through the C ABI: a replay must give exactly what the same calls give when
issued one by one, on every replay, with other work of the program and synchronisations in between."""
import numpy as np
import pytest

from acrotensor_amd import workloads
from gpu_helpers import to_tensor

pytestmark = pytest.mark.gpu


def bound_chain(at, wl):
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    for t in tensors.values():
        t.MoveToGPU()
    return tensors


def test_replays_of_a_fused_operator_apply_match_eager_launches(at, engine):
    wl = workloads.config4(E=301)
    tensors = bound_chain(at, wl)
    X, Y = tensors["X"], tensors["Y"]
    workloads.launch(wl, engine, tensors)                 # once eagerly: code object loaded, nothing left to allocate
    with at.recorded_launches() as seq:
        workloads.launch(wl, engine, tensors)
    for rep in range(4):
        X.Mult(-1.5)                                      # eager work between the replays
        at.synchronize()
        seq.launch()
        Y.MoveFromGPU()
        replayed = Y.data.copy()
        Y.MoveToGPU()
        Y.Set(0.0)
        workloads.launch(wl, engine, tensors)             # the same inputs, launched one by one
        Y.MoveFromGPU()
        assert np.array_equal(replayed, Y.data), rep
        assert np.abs(replayed).max() > 0
        Y.MoveToGPU()


def test_a_whole_pipeline_in_one_recording(at, engine):
    # node vector -> element vector -> mass apply -> node vector, plus a split contraction (two launches and a
    # scratch buffer) and an assignment that needs a zero fill first: seven launches recorded as one sequence
    dofs, nodes = workloads.hex_mesh_dof_map(4, 3, 2, 3)
    E = dofs.shape[0]
    wl = workloads.config4(E=E)
    tensors = bound_chain(at, wl)
    M = at.IndexMapping(nodes, dofs.size)
    M.map[:] = dofs.ravel()
    rng = np.random.default_rng(3)
    L, Lout = to_tensor(at, rng.uniform(-1, 1, nodes)), at.Tensor(nodes)
    n = 5000
    A, W, S = to_tensor(at, rng.uniform(0, 1, (n, 3, 3))), to_tensor(at, np.ones(n)), at.Tensor(3, 3)
    Dg, V = at.Tensor(6, 6), to_tensor(at, np.arange(1.0, 7.0))
    for t in (L, Lout, A, W, S, Dg, V):
        t.MoveToGPU()

    def pipeline():
        engine.FlatIndexedScatter(tensors["X"], L, M)
        workloads.launch(wl, engine, tensors)
        engine.FlatIndexedSumGather(Lout, tensors["Y"], M)
        engine("S_i_j = A_n_i_j B_n", S, A, W)
        engine("D_i_i = V_i", Dg, V)

    def results():
        out = []
        for t in (Lout, S, Dg):
            t.MoveFromGPU()
            out.append(t.data.copy())
            t.MoveToGPU()
        return out

    pipeline()
    eager = results()
    assert np.array_equal(eager[2], np.diag(np.arange(1.0, 7.0)))
    with at.recorded_launches() as seq:
        pipeline()
    for rep in range(3):
        for t in (Lout, S, Dg):
            t.Set(-3.0)                                   # eager work; every replay must overwrite all of it
        at.synchronize()
        seq.launch()
        for got, expected in zip(results(), eager):
            assert np.array_equal(got, expected), rep


def test_work_that_needs_the_host_is_refused_while_recording(at, engine):
    A, B = at.Tensor(8, 3), to_tensor(at, np.arange(24.0).reshape(8, 3))     # B is still on the host
    A.SwitchToGPU()
    with pytest.raises(at.AcroError, match="being recorded"):
        with at.recorded_launches():
            engine("A_e_i = B_e_i", A, B)                 # would have to copy B to the device
    # the recording was discarded and the stream is usable again
    engine("A_e_i = B_e_i", A, B)
    A.MoveFromGPU()
    assert np.array_equal(A.data, B.data)
    with pytest.raises(at.AcroError):
        at.recorded_launches().launch()                   # nothing recorded
