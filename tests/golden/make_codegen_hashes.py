"""Writes tests/golden/codegen_hashes.json: SHA-1 of the source that the generator emits for the five baseline
configurations (full sizes, intermediates transient and stored) and for one kernel of every other schedule.

The generator needs no device, so this runs anywhere the library is built.  tests/test_codegen_golden.py compares
against the file: a change of the generator that alters any emitted kernel has to be deliberate, and is recorded by
running this script again."""
import hashlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import acrotensor_amd as at                      # noqa: E402
from acrotensor_amd import workloads             # noqa: E402

CHAINS = {"cfg4": (workloads.config4, 262144), "cfg5": (workloads.config5, 65536)}
SINGLES = [
    ("cfg1", "S_i_j = A_n_i_j B_n", [(3, 3), (1 << 20, 3, 3), (1 << 20,)]),
    ("cfg3", "M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s",
     [(32768, 3, 3, 3, 3, 3, 3)] + [(4, 3)] * 6 + [(32768, 4, 4, 4)]),
    ("copy", "A_e_i = B_e_i", [(1 << 22, 16), (1 << 22, 16)]),
    ("matvec_lane_shared", "A_e_i = B_e_i_j C_e_j", [(1 << 15, 64), (1 << 15, 64, 64), (1 << 15, 64)]),
    ("matvec_row_sums", "A_e_i = B_e_i_j C_e_j", [(1 << 17, 27), (1 << 17, 27, 27), (1 << 17, 27)]),
    ("operator_mfma", "A_e_i = B_i_j X_e_j", [(1 << 18, 64), (64, 64), (1 << 18, 64)]),
    ("operator_components", "A_e_i_k = B_i_j X_e_j_k", [(1 << 16, 64, 3), (64, 64), (1 << 16, 64, 3)]),
    ("operator_entries_fastest", "A_i_e = B_i_j X_j_e", [(32, 1 << 18), (32, 32), (32, 1 << 18)]),
    ("copy_out_tile", "A_e_i = B_i_j X_e_j", [(1 << 21, 27), (27, 3), (1 << 21, 3)]),
    ("transpose", "A_i_j = B_j_i", [(8192, 8192), (8192, 8192)]),
    ("product_mfma_rows_in_pairs", "A_e_i_j = B_e_i_k C_e_k_j", [(4096, 64, 64), (4096, 64, 64), (4096, 64, 64)]),
    ("product_mfma_strips_through_lds", "A_e_i_j = B_e_i_k C_e_j_k", [(5546, 55, 55), (5546, 55, 55), (5546, 55, 55)]),
    ("product_mfma_tiled_batched", "A_e_i_j = B_e_i_k C_e_k_j", [(1024, 128, 128), (1024, 128, 128), (1024, 128, 128)]),
    ("product_mfma_tiled_plain", "A_i_j += B_k_i C_j_k", [(1000, 700), (333, 1000), (700, 333)]),
    ("product_mfma_tiled_shares", "A_i_j = B_n_i C_n_j", [(96, 80), (100000, 96), (100000, 80)]),
    ("row_reduction", "S_i = A_i_n", [(64,), (64, 1 << 20)]),
    ("dsetup", "D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j",
     [(16384, 3, 3, 10, 10, 10), (10, 10, 10), (16384, 10, 10, 10), (16384, 10, 10, 10), (16384, 10, 10, 10, 3, 3),
      (16384, 10, 10, 10, 3, 3)]),
]


def chain_source(factory, E, transient):
    small = factory(E=2)
    axes = {}
    for k, out, ins in small.kernels:
        lhs, rhs = k.replace("+=", "=").split("=")
        for token, name in zip([lhs.split()[0]] + rhs.split(), [out] + list(ins)):
            axes[name] = token.split("_")[1:]
    tensors = {}
    for name, arr in small.arrays.items():
        shape = list(arr.shape)
        if name in axes and "e" in axes[name]:
            shape[axes[name].index("e")] = E
        tensors[name] = at.Tensor(*shape)
    for name, (parent, idx) in small.slices.items():
        tensors[name] = at.SliceTensor(tensors[parent], *idx)
    for name in small.transient:
        tensors[name].SetTransient(transient)
    engine = at.TensorEngine("HIP")
    engine.BeginMultiKernelLaunch()
    for k, out, ins in small.kernels:
        engine(k, tensors[out], *[tensors[n] for n in ins])
    return engine.EndMultiKernelLaunchGetImplementation()


def all_sources():
    sources = {}
    for name, (factory, E) in CHAINS.items():
        sources[name + "_transient"] = chain_source(factory, E, True)
        sources[name + "_stored"] = chain_source(factory, E, False)
    engine = at.TensorEngine("HIP")
    for name, kernel, shapes in SINGLES:
        tensors = [at.Tensor(*s) for s in shapes]
        if name == "dsetup":
            tensors = tensors[:5] + [tensors[4]]          # Jinv twice
        sources[name] = engine.GetImplementation(kernel, tensors[0], *tensors[1:])
    return sources


def all_hashes():
    return {name: hashlib.sha1(src.encode()).hexdigest() for name, src in sorted(all_sources().items())}


if __name__ == "__main__":
    path = os.path.join(HERE, "codegen_hashes.json")
    with open(path, "w") as f:
        json.dump(all_hashes(), f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path)
