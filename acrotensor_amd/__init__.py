"""acrotensor_amd - host-side Python mirror of the Acrotensor API over the C ABI of the MI355X "HIP" backend.

The classes keep the names and call shapes of the reference's C++ API (``Tensor``, ``SliceTensor``,
``IndexMapping``, ``TensorEngine`` with ``TE("S_i_j = A_n_i_j B_n", S, A, B)``, ``MapToGPU`` / ``MoveToGPU`` /
``SwitchToGPU`` / ``MoveFromGPU``, ``BeginMultiKernelLaunch`` / ``EndMultiKernelLaunch``, the five non-contraction
operations); every call goes through ``libacrotensor_hip.so``.  Errors that the C++ API throws surface as
``AcroError``.  There is no host compute path in this package.
"""
from .api import (AcroError, IndexMapping, SliceTensor, Tensor, TensorEngine, describe_kernels, hip_event_timer,
                  get_stream, is_hip_ready, recorded_launches, set_pinned_host_allocation, set_stream, synchronize)

__all__ = ["AcroError", "IndexMapping", "SliceTensor", "Tensor", "TensorEngine", "describe_kernels",
           "get_stream", "hip_event_timer", "is_hip_ready", "recorded_launches", "set_pinned_host_allocation", "set_stream",
           "synchronize"]
