"""ctypes loader for libacrotensor_hip.so (the C ABI declared in include/acrotensor_hip.h).

The library is built in-tree by ``acrotensor_amd.build.build_library`` (hipcc, gfx950).  Loading fails loudly when
it is missing: there is no host fallback for any operation.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libacrotensor_hip.so")

c_int_p = ctypes.POINTER(ctypes.c_int)
c_double_p = ctypes.POINTER(ctypes.c_double)
c_size_t_p = ctypes.POINTER(ctypes.c_size_t)
handle = ctypes.c_void_p
handle_p = ctypes.POINTER(ctypes.c_void_p)

# name -> (restype, argtypes); every symbol that include/acrotensor_hip.h declares
SIGNATURES = {
    "acro_last_error": (ctypes.c_char_p, []),
    "acro_hip_is_ready": (ctypes.c_int, []),
    "acro_hip_synchronize": (ctypes.c_int, []),
    "acro_hip_set_stream": (ctypes.c_int, [ctypes.c_void_p]),
    "acro_hip_get_stream": (ctypes.c_void_p, []),
    "acro_hip_event_create": (ctypes.c_int, [handle_p]),
    "acro_hip_event_record": (ctypes.c_int, [handle]),
    "acro_tensor_set_pinned_host_allocation": (ctypes.c_int, [ctypes.c_int]),
    "acro_hip_graph_begin_capture": (ctypes.c_int, []),
    "acro_hip_graph_end_capture": (ctypes.c_int, [ctypes.POINTER(handle)]),
    "acro_hip_graph_abort_capture": (ctypes.c_int, []),
    "acro_hip_graph_launch": (ctypes.c_int, [handle]),
    "acro_hip_graph_destroy": (ctypes.c_int, [handle]),
    "acro_hip_event_elapsed_ms": (ctypes.c_int, [handle, handle, ctypes.POINTER(ctypes.c_float)]),
    "acro_hip_event_destroy": (ctypes.c_int, [handle]),
    "acro_tensor_create": (ctypes.c_int, [ctypes.c_int, c_int_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, handle_p]),
    "acro_tensor_create_slice": (ctypes.c_int, [handle, ctypes.c_int, c_int_p, handle_p]),
    "acro_tensor_destroy": (ctypes.c_int, [handle]),
    "acro_tensor_rank": (ctypes.c_int, [handle]),
    "acro_tensor_size": (ctypes.c_longlong, [handle]),
    "acro_tensor_dim": (ctypes.c_int, [handle, ctypes.c_int]),
    "acro_tensor_stride": (ctypes.c_longlong, [handle, ctypes.c_int]),
    "acro_tensor_data": (ctypes.c_void_p, [handle]),
    "acro_tensor_device_data": (ctypes.c_void_p, [handle]),
    "acro_tensor_reshape": (ctypes.c_int, [handle, ctypes.c_int, c_int_p]),
    "acro_tensor_retarget": (ctypes.c_int, [handle, ctypes.c_void_p, ctypes.c_void_p]),
    "acro_tensor_map_to_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_move_to_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_switch_to_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_unmap_from_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_move_from_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_switch_from_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_is_mapped_to_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_is_on_gpu": (ctypes.c_int, [handle]),
    "acro_tensor_set": (ctypes.c_int, [handle, ctypes.c_double]),
    "acro_tensor_mult": (ctypes.c_int, [handle, ctypes.c_double]),
    "acro_tensor_set_transient": (ctypes.c_int, [handle, ctypes.c_int]),
    "acro_index_mapping_create": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, handle_p]),
    "acro_index_mapping_destroy": (ctypes.c_int, [handle]),
    "acro_index_mapping_data": (ctypes.c_void_p, [handle]),
    "acro_index_mapping_compute_inverse": (ctypes.c_int, [handle]),
    "acro_index_mapping_inverse_data": (ctypes.c_void_p, [handle]),
    "acro_index_mapping_inverse_offsets": (ctypes.c_void_p, [handle]),
    "acro_engine_create": (ctypes.c_int, [ctypes.c_char_p, handle_p]),
    "acro_engine_destroy": (ctypes.c_int, [handle]),
    "acro_engine_set_executor_type": (ctypes.c_int, [handle, ctypes.c_char_p]),
    "acro_engine_contract": (ctypes.c_int, [handle, ctypes.c_char_p, handle, handle_p, ctypes.c_int]),
    "acro_engine_contract_no_alloc": (ctypes.c_int, [handle, ctypes.c_char_p, handle, handle_p, ctypes.c_int]),
    "acro_engine_begin_multi_kernel_launch": (ctypes.c_int, [handle]),
    "acro_engine_end_multi_kernel_launch": (ctypes.c_int, [handle]),
    "acro_engine_get_implementation": (ctypes.c_int, [handle, ctypes.c_char_p, handle, handle_p, ctypes.c_int,
                                                      ctypes.c_char_p, ctypes.c_size_t, c_size_t_p]),
    "acro_engine_end_multi_kernel_get_implementation": (ctypes.c_int, [handle, ctypes.c_char_p, ctypes.c_size_t, c_size_t_p]),
    "acro_engine_get_last_implementation": (ctypes.c_int, [handle, ctypes.c_char_p, ctypes.c_size_t, c_size_t_p]),
    "acro_engine_clear": (ctypes.c_int, [handle]),
    "acro_engine_batch_matrix_inverse": (ctypes.c_int, [handle, handle, handle]),
    "acro_engine_batch_matrix_det": (ctypes.c_int, [handle, handle, handle]),
    "acro_engine_batch_matrix_inv_det": (ctypes.c_int, [handle, handle, handle, handle]),
    "acro_engine_flat_indexed_scatter": (ctypes.c_int, [handle, handle, handle, handle]),
    "acro_engine_flat_indexed_sum_gather": (ctypes.c_int, [handle, handle, handle, handle]),
    "acro_hip_compile": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_char_p, c_size_t_p]),
    "acro_hip_compile_private_bytes": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int)]),
    "acro_describe_kernels": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(ctypes.c_char_p), c_int_p, c_int_p,
                                             ctypes.c_char_p, ctypes.c_size_t, c_size_t_p]),
}

_lib = None


def load():
    """Load the shared library once and set the prototypes of every declared entry point."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libacrotensor_hip.so is not built (%s missing): run `python -c 'import __graft_entry__ as g; "
                "g.build()'` or `make -C acrotensor_amd/csrc`; there is no host fallback." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib
