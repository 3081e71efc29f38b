"""The on-disk cache of compiled kernels: a second process-independent engine reuses the code object, and a damaged
cache file is replaced instead of failing the launch."""
import glob
import os

import numpy as np
import pytest

from gpu_helpers import to_tensor

pytestmark = pytest.mark.gpu


def test_damaged_cache_entry_is_recompiled(at, tmp_path, monkeypatch):
    monkeypatch.setenv("ACRO_HIP_CACHE_DIR", str(tmp_path))
    B = to_tensor(at, np.arange(35.0).reshape(7, 5))
    kernel = "A_e_i = B_e_i"
    first = at.TensorEngine("HIP")
    A = at.Tensor(7, 5)
    first(kernel, A, B)
    A.MoveFromGPU()
    assert np.array_equal(A.data, B.data)
    files = glob.glob(os.path.join(str(tmp_path), "*.hsaco"))
    assert len(files) == 1
    with open(files[0], "wb") as f:
        f.write(b"not a code object")
    second = at.TensorEngine("HIP")                 # a new engine reads the cache again
    A2 = at.Tensor(7, 5)
    second(kernel, A2, B)
    A2.MoveFromGPU()
    assert np.array_equal(A2.data, B.data)
    assert os.path.getsize(files[0]) > 100          # rewritten with a real code object
