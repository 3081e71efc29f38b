"""Adoption of a caller's stream (acro_hip_set_stream, the counterpart of the reference's setCudaContext,
util/CudaUtil.hpp:93-98, exercised by unittest/kernel/test_TensorEngine.cpp:149-185): everything the library
launches runs on the adopted stream, work queued before a switch precedes work queued after it, and the library's
own stream works again after the caller's stream has been handed back."""
import ctypes

import numpy as np
import pytest

from acrotensor_amd import workloads
from gpu_helpers import rel_err, to_tensor

pytestmark = pytest.mark.gpu
HIP_STREAM_NON_BLOCKING = 1


@pytest.fixture
def caller_stream():
    """A hipStream_t created by the test itself, the way an application would (default priority)."""
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipStreamCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreateWithFlags(ctypes.byref(stream), HIP_STREAM_NON_BLOCKING) == 0
    yield hip, stream
    assert hip.hipStreamSynchronize(stream) == 0
    assert hip.hipStreamDestroy(stream) == 0


def run_everything(at, engine, checker, seed):
    """A fused chain, a single contraction, a split contraction, a batched inverse / determinant, a scatter and a
    sum-gather, a fill and a scale; returns the worst relative deviation from the checker (0 for the exact ones)."""
    print("caller stream: seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    worst = 0.0
    wl = workloads.config4(E=37, seed=seed)
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    workloads.launch(wl, engine, tensors)
    tensors["Y"].MoveFromGPU()
    worst = max(worst, rel_err(tensors["Y"].data, workloads.run_on_checker(wl, checker)["Y"]))

    A, B = rng.uniform(-1, 1, (6, 5)), rng.uniform(-1, 1, (5, 7))
    C = at.Tensor(6, 7)
    engine("C_i_k = A_i_j B_j_k", C, to_tensor(at, A), to_tensor(at, B))
    C.MoveFromGPU()
    expected = np.zeros((6, 7))
    checker.contract("C_i_k = A_i_j B_j_k", expected, A, B)
    worst = max(worst, rel_err(C.data, expected))

    n = 30011
    R = (rng.integers(0, 9, (n, 3, 3))).astype(np.float64)
    S = at.Tensor(3, 3)
    engine("S_i_j = A_n_i_j B_n", S, to_tensor(at, R), to_tensor(at, np.ones(n)))
    S.MoveFromGPU()
    assert np.array_equal(S.data, R.sum(axis=0))

    J = workloads.config2_inputs(E=5, Q=13, seed=seed)
    Jinv, Jdet = at.Tensor(5, 13, 3, 3), at.Tensor(5, 13)
    engine.BatchMatrixInvDet(Jinv, Jdet, to_tensor(at, J))
    Jinv.MoveFromGPU()
    Jdet.MoveFromGPU()
    ri, rd = checker.batch_matrix_inv_det(J)
    assert np.array_equal(Jinv.data, ri) and np.array_equal(Jdet.data, rd)

    dofs, nodes = workloads.hex_mesh_dof_map(3, 2, 2, 2)
    M = at.IndexMapping(nodes, dofs.size)
    M.map[:] = dofs.ravel()
    Lv = rng.integers(-5, 6, nodes).astype(np.float64)
    Ev, back = at.Tensor(dofs.size), at.Tensor(nodes)
    engine.FlatIndexedScatter(Ev, to_tensor(at, Lv), M)
    engine.FlatIndexedSumGather(back, Ev, M)
    Ev.MoveFromGPU()
    back.MoveFromGPU()
    assert np.array_equal(Ev.data, Lv[dofs.ravel()])
    assert np.array_equal(back.data, np.bincount(dofs.ravel(), minlength=nodes) * Lv)

    F = at.Tensor(1000)
    F.MoveToGPU()
    F.Set(3.0)
    F.Mult(-0.5)
    F.MoveFromGPU()
    assert np.array_equal(F.data, np.full(1000, -1.5))
    return worst


def test_work_runs_on_an_adopted_stream_and_on_the_own_stream_afterwards(at, engine, checker, caller_stream):
    hip, stream = caller_stream
    own = at.get_stream()
    assert own and own != stream.value
    assert run_everything(at, engine, checker, 1) <= 1e-12
    at.set_stream(stream)
    assert at.get_stream() == stream.value
    assert run_everything(at, engine, checker, 2) <= 1e-12
    at.set_stream(None)
    assert at.get_stream() == own
    assert run_everything(at, engine, checker, 3) <= 1e-12


def test_work_queued_before_a_switch_precedes_work_queued_after_it(at, engine, caller_stream):
    # a long chain of dependent launches on one stream, then its result is read by a kernel launched right after the
    # switch, without any synchronisation by the host in between; both directions
    hip, stream = caller_stream
    n = 1 << 22
    X = at.Tensor(n)
    X.data[...] = 1.0
    Y = at.Tensor(n)
    X.MoveToGPU()
    Y.MoveToGPU()
    engine("Y_i = X_i", Y, X)                      # compile and load before the timing-sensitive part
    at.synchronize()
    expected = 1.0
    for direction in (stream, None, stream, None):
        for _ in range(40):
            X.Mult(1.0078125)                       # exact in fp64 for this many steps
            expected *= 1.0078125
        at.set_stream(direction)
        engine("Y_i = X_i", Y, X)                  # reads X on the other stream
        Y.MoveFromGPU()
        assert Y.data.min() == expected and Y.data.max() == expected
        Y.MoveToGPU()
    assert at.get_stream() != stream.value


def test_recording_on_an_adopted_stream(at, engine, caller_stream):
    # a launch sequence recorded while a caller's stream is adopted replays there; the stream cannot be changed
    # while the recording is open
    hip, stream = caller_stream
    wl = workloads.config4(E=19)
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    for t in tensors.values():
        t.MoveToGPU()
    at.set_stream(stream)
    try:
        workloads.launch(wl, engine, tensors)
        tensors["Y"].MoveFromGPU()
        eager = tensors["Y"].data.copy()
        tensors["Y"].MoveToGPU()
        with at.recorded_launches() as seq:
            workloads.launch(wl, engine, tensors)
            with pytest.raises(at.AcroError, match="being recorded"):
                at.set_stream(None)
        for rep in range(3):
            tensors["Y"].Set(0.0)
            at.synchronize()
            seq.launch()
            tensors["Y"].MoveFromGPU()
            assert np.array_equal(tensors["Y"].data, eager), rep
            tensors["Y"].MoveToGPU()
        del seq
    finally:
        at.set_stream(None)
