"""Synthetic workloads of the five baseline configurations, shared by the benchmark, the smoke test and the tests.

Inputs come from a counter-based generator (splitmix64 of seed, tensor number and flat index), so any element of
any tensor can be produced on its own, identically on every machine, without materialising anything else.

A workload is a list of kernels ``(kernel string, output name, input names)`` over named arrays; it can be run on
the HIP engine (``run_on_engine``) and handed, as plain numpy arrays, to whatever checker a test uses.
"""
import numpy as np

_MASK = (1 << 64) - 1


def _splitmix64_inplace(z):
    """splitmix64 finaliser applied in place to a uint64 array (arithmetic wraps modulo 2^64)."""
    z += np.uint64(0x9E3779B97F4A7C15)
    z ^= z >> np.uint64(30)
    z *= np.uint64(0xBF58476D1CE4E5B9)
    z ^= z >> np.uint64(27)
    z *= np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    return z


def counter_uniform(seed, tensor_id, shape, lo=0.0, hi=1.0, first=0):
    """fp64 array of ``shape``: entry with flat index i is uniform in [lo, hi), a pure function of (seed, tensor_id, first+i)."""
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float64)
    with np.errstate(over="ignore"):
        base = _splitmix64_inplace(np.array([np.uint64(seed) * np.uint64(0x1000003) + np.uint64(tensor_id)],
                                            dtype=np.uint64))[0]
        chunk = 1 << 18                                   # a few passes over 2 MiB at a time stay in cache
        for start in range(0, n, chunk):
            stop = min(n, start + chunk)
            bits = np.arange(first + start, first + stop, dtype=np.uint64)
            bits *= np.uint64(0x9E3779B97F4A7C15)
            bits += base
            _splitmix64_inplace(bits)
            bits >>= np.uint64(11)
            u = out[start:stop]
            u[...] = bits                                 # exact: 53 bits
            u *= 1.0 / 9007199254740992.0
            if not (lo == 0.0 and hi == 1.0):
                u *= (hi - lo)
                u += lo
    return out.reshape(shape)


class Workload:
    """Named arrays plus an ordered list of kernels; ``slices`` maps a name to (parent name, leading indices)."""

    def __init__(self, name, arrays, kernels, transient=(), slices=None, outputs=(), dof=0, algorithmic_bytes=0,
                 flops=0, seed=0):
        self.name = name
        self.arrays = arrays          # name -> numpy array (inputs filled, outputs zero)
        self.kernels = kernels        # list of (kernel string, out name, [in names])
        self.transient = tuple(transient)
        self.slices = slices or {}
        self.outputs = tuple(outputs)
        self.dof = dof
        self.algorithmic_bytes = algorithmic_bytes
        self.flops = flops
        self.seed = seed
        written = {out for _, out, _ in kernels}
        written |= {self.slices[n][0] for n in written if n in self.slices}
        self.inputs = tuple(n for n in arrays if n not in written)   # arrays that carry data into the first kernel

    def view(self, name, arrays=None):
        arrays = self.arrays if arrays is None else arrays
        if name in self.slices:
            parent, idx = self.slices[name]
            return arrays[parent][tuple(idx)]
        return arrays[name]


def bind_to_engine(workload, at, transient=True, inputs_only=False):
    """Create engine tensors for a workload; returns name -> Tensor (slices as SliceTensor of their parent).
    ``inputs_only``: the host buffers of tensors that the kernels write are left as allocated (large benchmarks)."""
    tensors = {}
    for name, arr in workload.arrays.items():
        t = at.Tensor(*arr.shape)
        if not inputs_only or name in workload.inputs:
            t.data[...] = arr
        tensors[name] = t
    for name, (parent, idx) in workload.slices.items():
        tensors[name] = at.SliceTensor(tensors[parent], *idx)
    for name in workload.transient:
        tensors[name].SetTransient(bool(transient))
    return tensors


def bind_to_engine_repeated(workload, at, engine, times, transient=True, index="e"):
    """Engine tensors for ``times`` copies of the workload laid end to end along the index called ``index`` (the
    element index), built on the device: inputs that carry the index are uploaded once and repeated there by a
    broadcasting kernel, tensors that the kernels write only get device memory.  For benchmarks at sizes whose
    inputs would take minutes to generate and upload (configs[4]: 4.7 GB of geometric factors); timings do not
    depend on the values.  Returns name -> Tensor."""
    axes = {}
    for k, out, ins in workload.kernels:
        lhs, rhs = k.replace("+=", "=").replace("-=", "=").split("=")
        for token, name in zip([lhs.split()[0]] + rhs.split(), [out] + list(ins)):
            axes[name] = token.split("_")[1:]
    tensors = {}
    for name, arr in workload.arrays.items():
        names = axes.get(name)
        if names is None or index not in names:
            t = at.Tensor(*arr.shape)                        # invariant operand (basis matrices)
            t.data[...] = arr
            t.MoveToGPU()
        elif name in workload.inputs:
            if names.index(index) != 0:
                raise ValueError("inputs must carry the repeated index first")
            small = at.Tensor(*arr.shape)
            small.data[...] = arr
            t = at.Tensor(times, *arr.shape)
            t.SwitchToGPU()
            letters = ["a%d" % d for d in range(arr.ndim)]
            engine("R_t_%s = S_%s" % ("_".join(letters), "_".join(letters)), t, small)
            t.Reshape(times * arr.shape[0], *arr.shape[1:])
        else:
            axis = names.index(index)
            t = at.Tensor(*[n * times if d == axis else n for d, n in enumerate(arr.shape)])
            t.SwitchToGPU()
        tensors[name] = t
    for name, (parent, idx) in workload.slices.items():
        tensors[name] = at.SliceTensor(tensors[parent], *idx)
    for name in workload.transient:
        tensors[name].SetTransient(bool(transient))
    return tensors


def launch(workload, engine, tensors):
    """One pass of the workload: a single kernel call, or one multi-kernel launch for a chain."""
    if len(workload.kernels) == 1:
        k, out, ins = workload.kernels[0]
        engine(k, tensors[out], *[tensors[n] for n in ins])
        return
    engine.BeginMultiKernelLaunch()
    for k, out, ins in workload.kernels:
        engine(k, tensors[out], *[tensors[n] for n in ins])
    engine.EndMultiKernelLaunch()


def run_on_checker(workload, checker):
    """Run the kernels one after the other on a checker with a ``contract(kernel, out, *ins)`` method (numpy arrays,
    in place).  Returns name -> array."""
    arrays = {k: v.copy() for k, v in workload.arrays.items()}
    for k, out, ins in workload.kernels:
        o = workload.view(out, arrays)
        if not o.flags["C_CONTIGUOUS"]:
            raise ValueError("slice outputs must be contiguous")
        checker.contract(k, o, *[np.ascontiguousarray(workload.view(n, arrays)) for n in ins])
    return arrays


# ------------------------------------------------------------------------------------------- the five configs

def config1(n=1 << 20, seed=0xAC21):
    """README batched reduction: S_i_j = A_n_i_j B_n, A[n,3,3] ~ U[0,1), B == 1."""
    arrays = {"A": counter_uniform(seed, 0, (n, 3, 3)), "B": np.ones(n), "S": np.zeros((3, 3))}
    return Workload("cfg1_batched_reduction", arrays, [("S_i_j = A_n_i_j B_n", "S", ["A", "B"])], outputs=("S",),
                    algorithmic_bytes=(n * 9 + n + 9) * 8, flops=2 * 9 * n, seed=seed)


def config2_inputs(E=65536, Q=64, seed=0xAC22):
    """Batched 3x3 Jacobians J = I + 0.1 U[-1,1)."""
    J = 0.1 * counter_uniform(seed, 0, (E, Q, 3, 3), -1.0, 1.0)
    J += np.eye(3)
    return J


def config3(E=32768, seed=0xAC23):
    """p=2 hex mass matrix full assembly (one 7-operand kernel, 10 loops)."""
    arrays = {"B": counter_uniform(seed, 0, (4, 3), -1.0, 1.0), "W": counter_uniform(seed, 1, (E, 4, 4, 4), 0.5, 1.5),
              "M": np.zeros((E, 3, 3, 3, 3, 3, 3))}
    k = "M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s"
    return Workload("cfg3_mass_assembly_p2", arrays, [(k, "M", ["B"] * 6 + ["W"])], outputs=("M",),
                    algorithmic_bytes=E * (64 + 729) * 8 + 96, flops=E * 729 * 64 * 7, seed=seed)


def config4(E=262144, seed=0xAC24, Q=5, P=4):
    """Sum-factorised hex mass operator apply as a 7-kernel chain (degree p = P - 1 with Q points per direction; the
    baseline configuration is p=3: Q, P = 5, 4)."""
    arrays = {
        "B": counter_uniform(seed, 0, (Q, P), -1.0, 1.0),
        "X": counter_uniform(seed, 1, (E, P, P, P), -1.0, 1.0),
        "D": counter_uniform(seed, 2, (E, Q, Q, Q), 0.5, 1.5),
        "T1": np.zeros((E, Q, P, P)), "T2": np.zeros((E, Q, Q, P)), "T3": np.zeros((E, Q, Q, Q)),
        "U": np.zeros((E, Q, Q, Q)), "V1": np.zeros((E, P, Q, Q)), "V2": np.zeros((E, P, P, Q)),
        "Y": np.zeros((E, P, P, P)),
    }
    kernels = [
        ("T1_e_q_j_k = B_q_i X_e_i_j_k", "T1", ["B", "X"]),
        ("T2_e_q_r_k = B_r_j T1_e_q_j_k", "T2", ["B", "T1"]),
        ("T3_e_q_r_s = B_s_k T2_e_q_r_k", "T3", ["B", "T2"]),
        ("U_e_q_r_s = D_e_q_r_s T3_e_q_r_s", "U", ["D", "T3"]),
        ("V1_e_i_r_s = B_q_i U_e_q_r_s", "V1", ["B", "U"]),
        ("V2_e_i_j_s = B_r_j V1_e_i_r_s", "V2", ["B", "V1"]),
        ("Y_e_i_j_k = B_s_k V2_e_i_j_s", "Y", ["B", "V2"]),
    ]
    flops_per_element = 2 * Q * P * (P * P + Q * P + Q * Q) * 2 + Q ** 3    # three stages each way + the pointwise product
    return Workload("cfg4_mass_apply_p%d" % (P - 1), arrays, kernels, transient=("T1", "T2", "T3", "U", "V1", "V2"),
                    outputs=("Y",), dof=E * P ** 3, algorithmic_bytes=E * (P ** 3 + Q ** 3 + P ** 3) * 8,
                    flops=E * flops_per_element, seed=seed)


def config5(E=65536, seed=0xAC25, Q=10, P=8):
    """p=7 sum-factorised hex diffusion operator apply: gradient, pointwise 3x3 apply, transposed gradient."""
    A = counter_uniform(seed, 3, (E, Q, Q, Q, 3, 3), -1.0, 1.0)
    D = np.einsum("...ik,...jk->...ij", A, A)
    D += 0.5 * np.eye(3)
    del A
    arrays = {
        "B": counter_uniform(seed, 0, (Q, P), -1.0, 1.0),
        "G": counter_uniform(seed, 1, (Q, P), -1.0, 1.0),
        "X": counter_uniform(seed, 2, (E, P, P, P), -1.0, 1.0),
        "D": np.ascontiguousarray(D),
        "T1g": np.zeros((E, Q, P, P)), "T1b": np.zeros((E, Q, P, P)),
        "T2a": np.zeros((E, Q, Q, P)), "T2b": np.zeros((E, Q, Q, P)), "T2c": np.zeros((E, Q, Q, P)),
        "U": np.zeros((3, E, Q, Q, Q)), "Z": np.zeros((3, E, Q, Q, Q)),
        "V1a": np.zeros((E, P, Q, Q)), "V1b": np.zeros((E, P, Q, Q)), "V1c": np.zeros((E, P, Q, Q)),
        "V2a": np.zeros((E, P, P, Q)), "V2b": np.zeros((E, P, P, Q)), "V2c": np.zeros((E, P, P, Q)),
        "Y": np.zeros((E, P, P, P)),
    }
    slices = {"U0": ("U", (0,)), "U1": ("U", (1,)), "U2": ("U", (2,)),
              "Z0": ("Z", (0,)), "Z1": ("Z", (1,)), "Z2": ("Z", (2,))}
    kernels = [
        ("T1g_e_q_j_k = G_q_i X_e_i_j_k", "T1g", ["G", "X"]),
        ("T1b_e_q_j_k = B_q_i X_e_i_j_k", "T1b", ["B", "X"]),
        ("T2a_e_q_r_k = B_r_j T1g_e_q_j_k", "T2a", ["B", "T1g"]),
        ("T2b_e_q_r_k = G_r_j T1b_e_q_j_k", "T2b", ["G", "T1b"]),
        ("T2c_e_q_r_k = B_r_j T1b_e_q_j_k", "T2c", ["B", "T1b"]),
        ("U0_e_q_r_s = B_s_k T2a_e_q_r_k", "U0", ["B", "T2a"]),
        ("U1_e_q_r_s = B_s_k T2b_e_q_r_k", "U1", ["B", "T2b"]),
        ("U2_e_q_r_s = G_s_k T2c_e_q_r_k", "U2", ["G", "T2c"]),
        ("Z_m_e_q_r_s = D_e_q_r_s_m_n U_n_e_q_r_s", "Z", ["D", "U"]),
        ("V1a_e_i_r_s = G_q_i Z0_e_q_r_s", "V1a", ["G", "Z0"]),
        ("V1b_e_i_r_s = B_q_i Z1_e_q_r_s", "V1b", ["B", "Z1"]),
        ("V1c_e_i_r_s = B_q_i Z2_e_q_r_s", "V1c", ["B", "Z2"]),
        ("V2a_e_i_j_s = B_r_j V1a_e_i_r_s", "V2a", ["B", "V1a"]),
        ("V2b_e_i_j_s = G_r_j V1b_e_i_r_s", "V2b", ["G", "V1b"]),
        ("V2c_e_i_j_s = B_r_j V1c_e_i_r_s", "V2c", ["B", "V1c"]),
        ("Y_e_i_j_k = B_s_k V2a_e_i_j_s", "Y", ["B", "V2a"]),
        ("Y_e_i_j_k += B_s_k V2b_e_i_j_s", "Y", ["B", "V2b"]),
        ("Y_e_i_j_k += G_s_k V2c_e_i_j_s", "Y", ["G", "V2c"]),
    ]
    transient = ("T1g", "T1b", "T2a", "T2b", "T2c", "U", "Z", "V1a", "V1b", "V1c", "V2a", "V2b", "V2c")
    flops_per_elem = 2 * (2 * Q * P * P * P + 3 * Q * Q * P * P + 3 * Q * Q * Q * P) * 2 + Q ** 3 * 9 * 2
    return Workload("cfg5_diffusion_apply_p7", arrays, kernels, transient=transient, slices=slices, outputs=("Y",),
                    dof=E * P ** 3, algorithmic_bytes=E * (P ** 3 + 9 * Q ** 3 + P ** 3) * 8,
                    flops=E * flops_per_elem, seed=seed)


def hex_mesh_dof_map(nx, ny, nz, p):
    """Element-to-node numbering of a structured nx x ny x nz hexahedral mesh of continuous degree-p elements:
    int32 array [E, p+1, p+1, p+1] of node numbers in [0, (nx p + 1)(ny p + 1)(nz p + 1)).  This is the IndexMapping an
    FE code uses with FlatIndexedScatter (node vector -> element vector) before an operator apply and with
    FlatIndexedSumGather (element vector -> node vector) after it (reference ops/NonContractionOps.hpp:27-31)."""
    n1 = p + 1
    gx, gy, gz = nx * p + 1, ny * p + 1, nz * p + 1
    ex, ey, ez = np.meshgrid(np.arange(nx), np.arange(ny), np.arange(nz), indexing="ij")
    base = ((ex * p) * gy + ey * p) * gz + ez * p                      # node of local (0, 0, 0), shape [nx, ny, nz]
    li, lj, lk = np.meshgrid(np.arange(n1), np.arange(n1), np.arange(n1), indexing="ij")
    local = (li * gy + lj) * gz + lk                                  # offsets of the local nodes
    dofs = base.reshape(-1, 1, 1, 1) + local[None]
    return dofs.astype(np.int32), gx * gy * gz
