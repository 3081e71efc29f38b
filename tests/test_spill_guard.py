"""Matrix-core kernels that the compiler can only fit with private memory (register spills) are never launched:
the check reads the kernel descriptors of the code object at compile time (no device needed), compiles a kernel that
fails it once more with the schedule's register-relief switch, and replaces it by a schedule without the matrix cores
if that does not help.  ACRO_HIP_TEST_PRIVATE_BYTES="first,second" stands for what the two compilations report, so
both branches run here with kernels that do not spill."""
import ctypes

import numpy as np
import pytest

import acrotensor_amd as at
from acrotensor_amd import _capi
from gpu_helpers import rel_err, run_single

OPERATOR = ("A_e_i = B_i_j X_e_j", [(500, 64), (64, 64), (500, 64)])
# the operator whose kernel was once seen to spill: 1 110 rows (370 points x 3 derivatives) by 52 columns, applied in
# blocks of rows, with the vector's components between the result's row indices
JACOBIANS = ("J_e_q_m_n = X_e_i_m G_q_i_n", [(400, 370, 3, 3), (400, 52, 3), (370, 52, 3)])
GRAM = ("A_i_j = B_e_i C_e_j", [(32, 32), (5000, 32), (5000, 32)])

WITH_PRIVATE_ARRAY = b"""extern "C" __global__ void keeps_an_array(double *out, const int *idx)
{
    double a[64];
    for (int i = 0; i < 64; ++i) a[i] = out[i] * 2.0;
    double s = 0;
    for (int i = 0; i < 64; ++i) s += a[idx[i] & 63];
    out[threadIdx.x] = s;
}
extern "C" __global__ void keeps_nothing(double *out) { out[threadIdx.x] = 1.0; }
"""


def implementation(kernel, shapes):
    tensors = [at.Tensor(*s) for s in shapes]
    return at.TensorEngine("HIP").GetImplementation(kernel, *tensors)


def test_private_memory_is_read_from_the_code_object():
    lib = _capi.load()
    n = ctypes.c_int(-7)
    assert lib.acro_hip_compile_private_bytes(b"unit_private", WITH_PRIVATE_ARRAY, b"keeps_an_array", ctypes.byref(n)) == 0
    assert n.value >= 512                                          # the 64 doubles, at least
    assert lib.acro_hip_compile_private_bytes(b"unit_private", WITH_PRIVATE_ARRAY, b"keeps_nothing", ctypes.byref(n)) == 0
    assert n.value == 0
    assert lib.acro_hip_compile_private_bytes(b"unit_private", WITH_PRIVATE_ARRAY, b"absent", ctypes.byref(n)) != 0
    assert b"no kernel called absent" in lib.acro_last_error()


@pytest.mark.parametrize("kernel,shapes", [OPERATOR, JACOBIANS, GRAM])
def test_matrix_core_kernels_as_generated_have_no_private_memory(monkeypatch, kernel, shapes):
    monkeypatch.delenv("ACRO_HIP_TEST_PRIVATE_BYTES", raising=False)
    monkeypatch.setenv("ACRO_HIP_CACHE_DIR", "off")
    src = implementation(kernel, shapes)
    assert "__builtin_amdgcn_mfma_f64_16x16x4f64" in src and "refused" not in src
    lib = _capi.load()
    import re
    for name in re.findall(r"__global__[^\n]*?\bvoid\s+(\w+)\s*\(", src):
        n = ctypes.c_int(-1)
        assert lib.acro_hip_compile_private_bytes(b"unit_guard", src.encode(), name.encode(), ctypes.byref(n)) == 0
        assert n.value == 0, name


def test_a_spilling_operator_kernel_is_compiled_again_with_its_relief_switch(monkeypatch):
    monkeypatch.setenv("ACRO_HIP_TEST_PRIVATE_BYTES", "68,0")
    src = implementation(*OPERATOR)
    assert src.startswith("#define ACRO_KEEP_OPERATOR_IN_LDS 1\n")
    assert "operator schedule on the FP64 matrix cores" in src and "refused" not in src


def test_a_kernel_that_still_spills_is_replaced_by_a_schedule_without_matrix_cores(monkeypatch):
    monkeypatch.setenv("ACRO_HIP_TEST_PRIVATE_BYTES", "68,68")
    for kernel, shapes in (OPERATOR, JACOBIANS):
        src = implementation(kernel, shapes)
        assert "mfma" not in src.replace("matrix-core kernel", "") and "was refused: this is the schedule without the matrix cores" in src
        assert "#define ACRO_KEEP_OPERATOR_IN_LDS" not in src


def test_a_schedule_without_a_relief_switch_falls_back_at_once(monkeypatch):
    monkeypatch.setenv("ACRO_HIP_TEST_PRIVATE_BYTES", "68,0")
    src = implementation(*GRAM)
    assert "Gram schedule" not in src and "_partial needed private memory" in src and "__builtin_amdgcn_mfma" not in src


def _random(shape, seed):
    return np.random.default_rng(seed).uniform(-1.0, 1.0, shape)


@pytest.mark.gpu
@pytest.mark.parametrize("report", [None, "68,0", "68,68"], ids=["as-compiled", "relief", "refused"])
@pytest.mark.parametrize("case", [OPERATOR, JACOBIANS, GRAM], ids=["operator", "jacobians", "gram"])
def test_every_branch_of_the_guard_gives_the_reference_result(monkeypatch, checker, case, report):
    if not at.is_hip_ready():
        pytest.fail("GPU test selected but no HIP device is usable")
    if report is None:
        monkeypatch.delenv("ACRO_HIP_TEST_PRIVATE_BYTES", raising=False)
    else:
        monkeypatch.setenv("ACRO_HIP_TEST_PRIVATE_BYTES", report)
    kernel, shapes = case
    engine = at.TensorEngine("HIP")                                # its variants are decided under this setting
    ins = [_random(s, 17 + i) for i, s in enumerate(shapes[1:])]
    got, expected = run_single(at, engine, checker, kernel, np.zeros(shapes[0]), *ins)
    assert rel_err(got, expected) <= 1e-12
    src = engine.GetLastImplementation()
    assert ("was refused" in src) == (report == "68,68" or (report == "68,0" and case is GRAM))
    # integer-valued data: every schedule must be exact
    ints = [np.round(4 * a) for a in ins]
    got, expected = run_single(at, engine, checker, kernel, np.zeros(shapes[0]), *ints)
    assert np.array_equal(got, expected)
