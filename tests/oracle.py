"""ctypes access to the checkers: oracle/liboracle.so (plain-C restatement of the reference's CPU path) and, when
it has been built, oracle/_ref/libacro_ref.so (the reference itself compiled for the CPU).  Test infrastructure
only: nothing in the product imports this module."""
import ctypes
import os

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(_ROOT, "oracle", "liboracle.so")
REF_PATH = os.path.join(_ROOT, "oracle", "_ref", "libacro_ref.so")

_c_int_p = ctypes.POINTER(ctypes.c_int)
_c_dbl_p = ctypes.POINTER(ctypes.c_double)


class _Checker:
    """Common call shapes of liboracle.so (prefix acro_oracle_) and libacro_ref.so (prefix acro_ref_)."""

    def __init__(self, path, prefix):
        self.lib = ctypes.CDLL(path)
        self.prefix = prefix

    def _fn(self, name):
        return getattr(self.lib, self.prefix + name)

    def contract(self, kernel, out, *ins):
        """out (numpy float64, modified in place) <op>= contraction of ins, as the CPU interpreter computes it."""
        arrays = [out] + list(ins)
        for a in arrays:
            assert a.dtype == np.float64 and a.flags["C_CONTIGUOUS"]
        ranks = (ctypes.c_int * len(arrays))(*[a.ndim for a in arrays])
        dim_arrays = [(ctypes.c_int * a.ndim)(*a.shape) for a in arrays]
        dims = (_c_int_p * len(arrays))(*[ctypes.cast(d, _c_int_p) for d in dim_arrays])
        in_ptrs = (_c_dbl_p * max(1, len(ins)))(*[a.ctypes.data_as(_c_dbl_p) for a in ins])
        err = ctypes.create_string_buffer(512)
        fn = self._fn("contract")
        fn.restype = ctypes.c_int
        rc = fn(kernel.encode(), out.ctypes.data_as(_c_dbl_p), in_ptrs, len(ins), dims, ranks, err, len(err))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        return out

    def name_string(self, kernel):
        buf = ctypes.create_string_buffer(4096)
        rc = self._fn("name_string")(kernel.encode(), buf, ctypes.c_size_t(len(buf)))
        if rc != 0:
            raise RuntimeError("kernel string rejected: " + kernel)
        return buf.value.decode()

    def batch_matrix_inverse(self, A):
        m = A.shape[-1]
        n = A.size // (m * m)
        R = np.empty_like(A)
        rc = self._fn("batch_matrix_inverse")(R.ctypes.data_as(_c_dbl_p), A.ctypes.data_as(_c_dbl_p), m, ctypes.c_long(n))
        assert rc == 0
        return R

    def batch_matrix_det(self, A):
        m = A.shape[-1]
        n = A.size // (m * m)
        D = np.empty(A.shape[:-2], dtype=np.float64)
        rc = self._fn("batch_matrix_det")(D.ctypes.data_as(_c_dbl_p), A.ctypes.data_as(_c_dbl_p), m, ctypes.c_long(n))
        assert rc == 0
        return D

    def batch_matrix_inv_det(self, A):
        m = A.shape[-1]
        n = A.size // (m * m)
        R = np.empty_like(A)
        D = np.empty(A.shape[:-2], dtype=np.float64)
        rc = self._fn("batch_matrix_inv_det")(R.ctypes.data_as(_c_dbl_p), D.ctypes.data_as(_c_dbl_p),
                                              A.ctypes.data_as(_c_dbl_p), m, ctypes.c_long(n))
        assert rc == 0
        return R, D

    def index_mapping_inverse(self, M, domain_size):
        M = np.ascontiguousarray(M, dtype=np.int32)
        inv = np.empty(M.size, dtype=np.int32)
        off = np.empty(domain_size + 1, dtype=np.int32)
        self._fn("index_mapping_inverse")(M.ctypes.data_as(_c_int_p), domain_size, M.size, inv.ctypes.data_as(_c_int_p),
                                          off.ctypes.data_as(_c_int_p))
        return inv, off


class Oracle(_Checker):
    def __init__(self):
        super().__init__(ORACLE_PATH, "acro_oracle_")

    def scatter(self, Ain, M):
        M = np.ascontiguousarray(M, dtype=np.int32)
        out = np.empty(M.size, dtype=np.float64)
        self.lib.acro_oracle_flat_indexed_scatter(out.ctypes.data_as(_c_dbl_p), Ain.ctypes.data_as(_c_dbl_p),
                                                  M.ctypes.data_as(_c_int_p), M.size)
        return out

    def sum_gather(self, Ain, M, domain_size):
        M = np.ascontiguousarray(M, dtype=np.int32)
        out = np.empty(domain_size, dtype=np.float64)
        self.lib.acro_oracle_flat_indexed_sum_gather(out.ctypes.data_as(_c_dbl_p), domain_size,
                                                     Ain.ctypes.data_as(_c_dbl_p), M.ctypes.data_as(_c_int_p), M.size)
        return out


class Reference(_Checker):
    def __init__(self):
        super().__init__(REF_PATH, "acro_ref_")

    def scatter(self, Ain, M):
        M = np.ascontiguousarray(M, dtype=np.int32)
        out = np.empty(M.size, dtype=np.float64)
        self.lib.acro_ref_flat_indexed_scatter(out.ctypes.data_as(_c_dbl_p), Ain.ctypes.data_as(_c_dbl_p), Ain.size,
                                               M.ctypes.data_as(_c_int_p), M.size)
        return out

    def sum_gather(self, Ain, M, domain_size):
        M = np.ascontiguousarray(M, dtype=np.int32)
        out = np.empty(domain_size, dtype=np.float64)
        self.lib.acro_ref_flat_indexed_sum_gather(out.ctypes.data_as(_c_dbl_p), domain_size,
                                                  Ain.ctypes.data_as(_c_dbl_p), M.ctypes.data_as(_c_int_p), M.size)
        return out

    def describe(self, kernel, shapes):
        ranks = (ctypes.c_int * len(shapes))(*[len(s) for s in shapes])
        dim_arrays = [(ctypes.c_int * len(s))(*s) for s in shapes]
        dims = (_c_int_p * len(shapes))(*[ctypes.cast(d, _c_int_p) for d in dim_arrays])
        buf = ctypes.create_string_buffer(8192)
        rc = self.lib.acro_ref_describe(kernel.encode(), dims, ranks, len(shapes) - 1, buf, ctypes.c_size_t(len(buf)))
        if rc != 0:
            raise RuntimeError("reference rejected: " + kernel)
        return dict(item.split(":", 1) for item in buf.value.decode().split(";"))


def have_reference():
    return os.path.exists(REF_PATH)
