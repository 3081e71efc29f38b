"""Python mirror of acro::Tensor / SliceTensor / IndexMapping / TensorEngine over the C ABI."""
import ctypes
import json

import numpy as np

from . import _capi


class AcroError(RuntimeError):
    """Raised where the C++ API throws std::runtime_error (ACROBATIC_ASSERT, HIP and hipRTC failures)."""


def _check(code):
    if code != 0:
        raise AcroError(_capi.load().acro_last_error().decode("utf-8", "replace"))


def _int_array(values):
    values = [int(v) for v in values]
    return (ctypes.c_int * max(1, len(values)))(*values), len(values)


def is_hip_ready():
    return bool(_capi.load().acro_hip_is_ready())


def set_stream(hip_stream):
    """Adopt a caller's ``hipStream_t`` (an integer address or ``ctypes.c_void_p``); ``None`` hands it back and
    returns to the library's own stream."""
    _check(_capi.load().acro_hip_set_stream(hip_stream))


def get_stream():
    return _capi.load().acro_hip_get_stream()


def synchronize():
    _check(_capi.load().acro_hip_synchronize())


def set_pinned_host_allocation(flag=True):
    """Host buffers of tensors created from now on are page-locked (faster ``MoveToGPU`` / ``MoveFromGPU``)."""
    _check(_capi.load().acro_tensor_set_pinned_host_allocation(1 if flag else 0))


class Tensor:
    """Dense row-major fp64 tensor: ``Tensor(d0, d1, ...)``.  ``.data`` is a numpy view of the host buffer.
    ``hdata`` wraps a caller's numpy array, ``ddata`` / ``ongpu`` additionally a caller's device buffer."""

    def __init__(self, *dims, hdata=None, ddata=None, ongpu=False, _handle=None, _keep=None):
        self._lib = _capi.load()
        self._keep = _keep            # objects that must outlive this tensor (external buffer, slice parent)
        self._h = ctypes.c_void_p()
        if _handle is not None:
            self._h = _handle
        elif dims:
            if len(dims) == 1 and isinstance(dims[0], (list, tuple)):
                dims = tuple(dims[0])
            arr, n = _int_array(dims)
            hptr = None
            if hdata is not None:
                if not (isinstance(hdata, np.ndarray) and hdata.dtype == np.float64 and hdata.flags["C_CONTIGUOUS"]):
                    raise AcroError("hdata must be a C-contiguous float64 numpy array")
                self._keep = hdata
                hptr = hdata.ctypes.data_as(ctypes.c_void_p)
            # ddata: address of an existing device buffer of the caller (with hdata only), ongpu: it holds the
            # current data (the reference's Tensor(dims, hdata, ddata, ongpu), tensor/Tensor.cpp:166-202)
            dptr = ctypes.c_void_p(int(ddata)) if ddata else None
            _check(self._lib.acro_tensor_create(n, arr, hptr, dptr, 1 if ongpu else 0, ctypes.byref(self._h)))
        else:
            raise AcroError("A tensor needs at least one dimension.")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.acro_tensor_destroy(h)

    # shape ---------------------------------------------------------------------------------------------
    def GetRank(self):
        return self._lib.acro_tensor_rank(self._h)

    def GetSize(self):
        return self._lib.acro_tensor_size(self._h)

    def GetDim(self, d):
        return self._lib.acro_tensor_dim(self._h, d)

    def GetStride(self, d):
        return self._lib.acro_tensor_stride(self._h, d)

    @property
    def dims(self):
        return tuple(self.GetDim(d) for d in range(self.GetRank()))

    def Reshape(self, *dims):
        arr, n = _int_array(dims)
        _check(self._lib.acro_tensor_reshape(self._h, n, arr))

    # data ----------------------------------------------------------------------------------------------
    @property
    def data(self):
        """numpy view (shape = dims) of the host buffer; valid while this object lives."""
        ptr = self._lib.acro_tensor_data(self._h)
        flat = np.ctypeslib.as_array(ctypes.cast(ptr, _capi.c_double_p), shape=(self.GetSize(),))
        return flat.reshape(self.dims)

    def GetDeviceData(self):
        return self._lib.acro_tensor_device_data(self._h)

    def Set(self, value):
        _check(self._lib.acro_tensor_set(self._h, float(value)))

    def Mult(self, factor):
        _check(self._lib.acro_tensor_mult(self._h, float(factor)))

    def SetTransient(self, flag=True):
        _check(self._lib.acro_tensor_set_transient(self._h, 1 if flag else 0))

    # residency -----------------------------------------------------------------------------------------
    def MapToGPU(self):
        _check(self._lib.acro_tensor_map_to_gpu(self._h))

    def MoveToGPU(self):
        _check(self._lib.acro_tensor_move_to_gpu(self._h))

    def SwitchToGPU(self):
        _check(self._lib.acro_tensor_switch_to_gpu(self._h))

    def UnmapFromGPU(self):
        _check(self._lib.acro_tensor_unmap_from_gpu(self._h))

    def MoveFromGPU(self):
        _check(self._lib.acro_tensor_move_from_gpu(self._h))

    def SwitchFromGPU(self):
        _check(self._lib.acro_tensor_switch_from_gpu(self._h))

    def IsMappedToGPU(self):
        return bool(self._lib.acro_tensor_is_mapped_to_gpu(self._h))

    def IsOnGPU(self):
        return bool(self._lib.acro_tensor_is_on_gpu(self._h))


class SliceTensor(Tensor):
    """View of ``parent`` at fixed leading indices: ``SliceTensor(T, i0, i1, ...)``."""

    def __init__(self, parent, *indices):
        lib = _capi.load()
        h = ctypes.c_void_p()
        arr, n = _int_array(indices)
        _check(lib.acro_tensor_create_slice(parent._h, n, arr, ctypes.byref(h)))
        super().__init__(_handle=h, _keep=parent)


class IndexMapping:
    """Map from a range of ``range_size`` entries into a domain of ``domain_size`` entries; ``.map`` is a numpy view."""

    def __init__(self, domain_size, range_size):
        self._lib = _capi.load()
        self._h = ctypes.c_void_p()
        self.domain_size, self.range_size = int(domain_size), int(range_size)
        _check(self._lib.acro_index_mapping_create(self.domain_size, self.range_size, ctypes.byref(self._h)))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.acro_index_mapping_destroy(h)

    @property
    def map(self):
        ptr = self._lib.acro_index_mapping_data(self._h)
        return np.ctypeslib.as_array(ctypes.cast(ptr, _capi.c_int_p), shape=(self.range_size,))

    def ComputeInverse(self):
        _check(self._lib.acro_index_mapping_compute_inverse(self._h))

    @property
    def inverse(self):
        p = self._lib.acro_index_mapping_inverse_data(self._h)
        o = self._lib.acro_index_mapping_inverse_offsets(self._h)
        if not p or not o:
            raise AcroError("Trying to access inverse mapping before the inverse is computed.")
        inv = np.ctypeslib.as_array(ctypes.cast(p, _capi.c_int_p), shape=(self.range_size,))
        off = np.ctypeslib.as_array(ctypes.cast(o, _capi.c_int_p), shape=(self.domain_size + 1,))
        return inv, off


def _fetch_string(call):
    needed = ctypes.c_size_t(0)
    _check(call(None, 0, ctypes.byref(needed)))
    buf = ctypes.create_string_buffer(needed.value + 1)
    _check(call(buf, len(buf), ctypes.byref(needed)))
    return buf.value.decode("utf-8", "replace")


class TensorEngine:
    """``TE = TensorEngine("HIP"); TE("S_i_j = A_n_i_j B_n", S, A, B)``."""

    def __init__(self, exec_type="HIP"):
        self._lib = _capi.load()
        self._h = ctypes.c_void_p()
        _check(self._lib.acro_engine_create(exec_type.encode(), ctypes.byref(self._h)))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.acro_engine_destroy(h)

    def SetExecutorType(self, exec_type):
        _check(self._lib.acro_engine_set_executor_type(self._h, exec_type.encode()))

    @staticmethod
    def _handles(tensors):
        arr = (ctypes.c_void_p * max(1, len(tensors)))(*[t._h for t in tensors])
        return arr, len(tensors)

    def __call__(self, kernel, out, *inputs):
        arr, n = self._handles(inputs)
        _check(self._lib.acro_engine_contract(self._h, kernel.encode(), out._h, arr, n))

    def contract_no_alloc(self, kernel, out, *inputs):
        """The same as calling the engine, for callers that cannot allocate: tensors must be resident on the device
        and the kernel must have run once through the ordinary call; scratch memory comes from a fixed array."""
        arr, n = self._handles(inputs)
        _check(self._lib.acro_engine_contract_no_alloc(self._h, kernel.encode(), out._h, arr, n))

    def GetImplementation(self, kernel, out, *inputs):
        arr, n = self._handles(inputs)
        return _fetch_string(lambda buf, size, needed: self._lib.acro_engine_get_implementation(
            self._h, kernel.encode(), out._h, arr, n, buf, size, needed))

    def GetLastImplementation(self):
        return _fetch_string(lambda buf, size, needed: self._lib.acro_engine_get_last_implementation(
            self._h, buf, size, needed))

    def BeginMultiKernelLaunch(self):
        _check(self._lib.acro_engine_begin_multi_kernel_launch(self._h))

    def EndMultiKernelLaunch(self):
        _check(self._lib.acro_engine_end_multi_kernel_launch(self._h))

    def EndMultiKernelLaunchGetImplementation(self):
        """End the capture without executing it; returns the fused kernel's source (needs no device)."""
        # The capture can only be ended once, so ask for a generous buffer first.
        size = 1 << 22
        buf = ctypes.create_string_buffer(size)
        needed = ctypes.c_size_t(0)
        _check(self._lib.acro_engine_end_multi_kernel_get_implementation(self._h, buf, size, ctypes.byref(needed)))
        return buf.value.decode("utf-8", "replace")

    def Clear(self):
        _check(self._lib.acro_engine_clear(self._h))

    def BatchMatrixInverse(self, Ainv, A):
        _check(self._lib.acro_engine_batch_matrix_inverse(self._h, Ainv._h, A._h))

    def BatchMatrixDet(self, Adet, A):
        _check(self._lib.acro_engine_batch_matrix_det(self._h, Adet._h, A._h))

    def BatchMatrixInvDet(self, Ainv, Adet, A):
        _check(self._lib.acro_engine_batch_matrix_inv_det(self._h, Ainv._h, Adet._h, A._h))

    def FlatIndexedScatter(self, Aout, Ain, M):
        _check(self._lib.acro_engine_flat_indexed_scatter(self._h, Aout._h, Ain._h, M._h))

    def FlatIndexedSumGather(self, Aout, Ain, M):
        _check(self._lib.acro_engine_flat_indexed_sum_gather(self._h, Aout._h, Ain._h, M._h))


def describe_kernels(kernels, shapes):
    """Parse and bind kernels on the host: ``shapes[k]`` lists the dims of kernel k's output then inputs."""
    lib = _capi.load()
    ks = (ctypes.c_char_p * len(kernels))(*[k.encode() for k in kernels])
    ranks, dims = [], []
    for per_kernel in shapes:
        for shp in per_kernel:
            ranks.append(len(shp))
            dims.extend(shp)
    r, _ = _int_array(ranks)
    d, _ = _int_array(dims)
    text = _fetch_string(lambda buf, size, needed: lib.acro_describe_kernels(len(kernels), ks, r, d, buf, size, needed))
    return json.loads(text)


class hip_event_timer:
    """Times work on the library's stream with HIP events: ``with hip_event_timer() as t: ...; t.ms``."""

    def __init__(self):
        self._lib = _capi.load()
        self._a, self._b = ctypes.c_void_p(), ctypes.c_void_p()
        _check(self._lib.acro_hip_event_create(ctypes.byref(self._a)))
        _check(self._lib.acro_hip_event_create(ctypes.byref(self._b)))
        self.ms = None

    def __enter__(self):
        _check(self._lib.acro_hip_event_record(self._a))
        return self

    def __exit__(self, *exc):
        _check(self._lib.acro_hip_event_record(self._b))
        ms = ctypes.c_float(0)
        _check(self._lib.acro_hip_event_elapsed_ms(self._a, self._b, ctypes.byref(ms)))
        self.ms = ms.value
        return False

    def __del__(self):
        for ev in (getattr(self, "_a", None), getattr(self, "_b", None)):
            if ev:
                self._lib.acro_hip_event_destroy(ev)


class recorded_launches:
    """Records everything the library would launch inside the ``with`` block (hipGraph) instead of executing it;
    ``launch()`` then enqueues the whole sequence with one call::

        apply()                                   # once, eagerly: loads kernels, allocates scratch
        with at.recorded_launches() as seq:
            apply()
        for _ in range(100):
            seq.launch()

    Tensors must be resident on the device and nothing inside the block may need the host (copies, allocation,
    synchronisation raise ``AcroError``; the recording is then discarded)."""

    def __init__(self):
        self._lib = _capi.load()
        self._g = ctypes.c_void_p()

    def __enter__(self):
        _check(self._lib.acro_hip_graph_begin_capture())
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is not None:
            self._lib.acro_hip_graph_abort_capture()
            return False
        _check(self._lib.acro_hip_graph_end_capture(ctypes.byref(self._g)))
        return False

    def launch(self):
        if not self._g:
            raise AcroError("nothing has been recorded")
        _check(self._lib.acro_hip_graph_launch(self._g))

    def __del__(self):
        g, self._g = getattr(self, "_g", None), None
        if g:
            self._lib.acro_hip_graph_destroy(g)
