"""The entry point that allocates nothing (acro_engine_contract_no_alloc) against the ordinary one, through the C ABI.

A split contraction (few outputs, long contraction) is the operation whose kernels keep per-workgroup partial sums
in scratch memory beyond their operands; the ordinary entry point allocates that buffer per kernel, the other one
takes it from a fixed array that every call on the device shares."""
import numpy as np
import pytest

from acrotensor_amd import workloads

pytestmark = pytest.mark.gpu
KERNEL = "S_i_j = A_n_i_j B_n"


def make(at, n, seed):
    A = at.Tensor(n, 3, 3)
    A.data[...] = workloads.counter_uniform(seed, 0, (n, 3, 3), -1.0, 1.0)
    B = at.Tensor(n)
    B.data[...] = workloads.counter_uniform(seed, 1, (n,), 0.5, 1.5)
    return A, B


def both_ways(at, engine, n, seed):
    print("split contraction without allocation: n =", n, "seed =", seed, flush=True)
    A, B = make(at, n, seed)
    expected_t, got_t = at.Tensor(3, 3), at.Tensor(3, 3)
    engine(KERNEL, expected_t, A, B)         # ordinary entry point: compiles, loads, allocates its own scratch
    got_t.data[...] = np.nan
    got_t.MoveToGPU()                        # residency is the caller's business here
    engine.contract_no_alloc(KERNEL, got_t, A, B)
    expected_t.MoveFromGPU()
    got_t.MoveFromGPU()
    return got_t.data.copy(), expected_t.data.copy(), A.data.sum(axis=0)


def test_two_calls_in_a_row_second_one_smaller(at, engine):
    # the second call finds the first one's partial sums in the shared array and must not pick any of them up
    for n, seed in ((1 << 20, 11), (100003, 12)):
        got, expected, _ = both_ways(at, engine, n, seed)
        assert np.array_equal(got, expected)             # same kernels, same fixed summation order: bit-identical


def test_accumulating_form_and_checker(at, engine, checker):
    n = 70001
    A, B = make(at, n, 13)
    S = at.Tensor(3, 3)
    S.data[...] = 0.0
    engine(KERNEL.replace(" = ", " += "), S, A, B)
    for _ in range(3):
        engine.contract_no_alloc(KERNEL.replace(" = ", " += "), S, A, B)
    S.MoveFromGPU()
    expected = np.zeros((3, 3))
    checker.contract(KERNEL, expected, A.data, B.data)
    assert np.abs(S.data - 4.0 * expected).max() <= 1e-12 * np.abs(4.0 * expected).max()


def test_refuses_what_would_allocate(at):
    engine = at.TensorEngine("HIP")        # an engine of its own: nothing it runs has been loaded before
    A, B = make(at, 5000, 14)
    S = at.Tensor(3, 3)
    # tensors not resident: moving them would allocate
    with pytest.raises(at.AcroError, match="must not allocate"):
        engine.contract_no_alloc(KERNEL, S, A, B)
    for t in (A, B, S):
        t.MoveToGPU()
    # resident, but this kernel at these extents has never been loaded
    with pytest.raises(at.AcroError, match="not loaded"):
        engine.contract_no_alloc(KERNEL, S, A, B)
    engine(KERNEL, S, A, B)
    engine.contract_no_alloc(KERNEL, S, A, B)
    S.MoveFromGPU()
    assert np.abs(S.data - np.einsum("nij,n->ij", A.data, B.data)).max() <= 1e-12 * np.abs(S.data).max()


def test_refuses_more_scratch_than_the_array_holds(at, engine):
    # 128 outputs x 512 shares of the contraction = 512 KiB of partial sums; the array holds 256 KiB
    n, m = 16384, 128
    A = at.Tensor(n, m)
    A.data[...] = workloads.counter_uniform(15, 0, (n, m), -1.0, 1.0)
    S = at.Tensor(m)
    engine("S_i = A_n_i", S, A)
    S.MoveFromGPU()
    expected = S.data.copy()
    S.MoveToGPU()
    with pytest.raises(at.AcroError, match="bytes of scratch memory"):
        engine.contract_no_alloc("S_i = A_n_i", S, A)
    # and the refusal leaves engine and device usable
    engine("S_i = A_n_i", S, A)
    S.MoveFromGPU()
    assert np.array_equal(S.data, expected)
    assert np.abs(expected - A.data.sum(axis=0)).max() <= 1e-12 * np.abs(expected).max()


def test_refused_inside_a_multi_kernel_launch(at, engine):
    # between Begin and End a call is only recorded, and the launch at End is an ordinary one that may allocate
    A, B = make(at, 3000, 16)
    S = at.Tensor(3, 3)
    for t in (A, B, S):
        t.MoveToGPU()
    engine(KERNEL, S, A, B)
    engine.BeginMultiKernelLaunch()
    try:
        with pytest.raises(at.AcroError, match="between BeginMultiKernelLaunch and EndMultiKernelLaunch"):
            engine.contract_no_alloc(KERNEL, S, A, B)
    finally:
        engine.EndMultiKernelLaunch()
    engine.contract_no_alloc(KERNEL, S, A, B)
    S.MoveFromGPU()
    assert np.abs(S.data - np.einsum("nij,n->ij", A.data, B.data)).max() <= 1e-12 * np.abs(S.data).max()
