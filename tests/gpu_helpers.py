"""Helpers of the GPU parity tests: run kernels on the HIP engine through the C ABI and on the checker."""
import numpy as np


def to_tensor(at, arr):
    t = at.Tensor(*arr.shape)
    t.data[...] = arr
    return t


def rel_err(got, expected):
    """max |got - expected| / max |expected| (the parity metric: relative to the largest entry of the tensor)."""
    scale = np.abs(expected).max()
    return np.abs(got - expected).max() / (scale if scale > 0 else 1.0)


def run_single(at, engine, checker, kernel, out_init, *ins):
    """Returns (engine result, checker result) of one kernel on the same inputs."""
    print("kernel:", kernel, "out", out_init.shape, "ins", [a.shape for a in ins], flush=True)
    out = to_tensor(at, out_init)
    tensors = [to_tensor(at, a) for a in ins]
    engine(kernel, out, *tensors)
    out.MoveFromGPU()
    expected = out_init.copy()
    checker.contract(kernel, expected, *[np.ascontiguousarray(a) for a in ins])
    return out.data.copy(), expected


def output_shape(kernel, shapes, default=3):
    lhs, rhs = kernel.replace("+=", "=").replace("-=", "=").split("=")
    sizes = {}
    for var, shp in zip(rhs.split(), shapes):
        for name, n in zip(var.split("_")[1:], shp):
            sizes[name] = n
    return tuple(sizes.get(n, default) for n in lhs.split()[0].split("_")[1:])
