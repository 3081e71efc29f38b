"""Writes the golden fixtures of this directory by running the REFERENCE ITSELF (oracle/_ref/libacro_ref.so, compiled
from the reference's sources by oracle/Makefile) on small seeded inputs.  Run in the build container, where the
reference sources are mounted:  python tests/golden/make_golden.py
Each .npz holds inputs and the reference's outputs only (data, no code)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from acrotensor_amd import workloads  # noqa: E402


def save(name, **arrays):
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)


def contract_fixture(ref, name, kernel, ins, out_init):
    expected = out_init.copy()
    ref.contract(kernel, expected, *ins)
    save(name, kind="contract", kernel=kernel, num_in=len(ins), out_init=out_init, expected=expected,
         **{"in%d" % i: a for i, a in enumerate(ins)})


def main():
    ref = oracle.Reference()
    rng = np.random.default_rng(20240)

    wl = workloads.config1(n=4096)
    contract_fixture(ref, "cfg1_reduction_n4096", wl.kernels[0][0], [wl.arrays["A"], wl.arrays["B"]], np.zeros((3, 3)))

    wl = workloads.config3(E=4)
    contract_fixture(ref, "cfg3_mass_assembly_E4", wl.kernels[0][0], [wl.arrays["B"]] * 6 + [wl.arrays["W"]],
                     np.zeros((4, 3, 3, 3, 3, 3, 3)))

    # one fixture per kernel of the mass-apply chain (E = 8), each fed with the reference's previous outputs
    wl = workloads.config4(E=8)
    arrays = workloads.run_on_checker(wl, ref)
    for n, (kernel, out, ins) in enumerate(wl.kernels):
        save("cfg4_mass_apply_E8_k%d" % n, kind="contract", kernel=kernel, num_in=len(ins),
             out_init=np.zeros_like(arrays[out]), expected=arrays[out],
             **{"in%d" % i: arrays[nm] for i, nm in enumerate(ins)})

    # the diffusion chain end to end (E = 2, Q = 5, P = 4): first and last kernels plus the pointwise apply
    wl = workloads.config5(E=2, Q=5, P=4)
    arrays = workloads.run_on_checker(wl, ref)
    for n in (0, 8):
        kernel, out, ins = wl.kernels[n]
        save("cfg5_diffusion_E2_k%d" % n, kind="contract", kernel=kernel, num_in=len(ins),
             out_init=np.zeros_like(wl.view(out, arrays)), expected=np.ascontiguousarray(wl.view(out, arrays)),
             **{"in%d" % i: np.ascontiguousarray(wl.view(nm, arrays)) for i, nm in enumerate(ins)})
    # whole workloads: inputs are regenerated from the counter-based generator (their sums are stored to detect
    # drift), outputs are the reference's
    for cfg, kwargs in (("config4", dict(E=8)), ("config5", dict(E=2, Q=5, P=4)), ("config3", dict(E=4)),
                        ("config1", dict(n=4096))):
        wl = getattr(workloads, cfg)(**kwargs)
        res = workloads.run_on_checker(wl, ref)
        names = sorted(kwargs)
        save("workload_%s" % cfg, kind="workload", config=cfg, arg_names=np.array(names),
             arg_values=np.array([kwargs[k] for k in names]),
             input_sums=np.array([wl.arrays[k].sum() for k in sorted(wl.arrays)]),
             **{"out_" + o: res[o] for o in wl.outputs})

    # accumulate forms and the reference interpreter's treatment of "-="
    B, C = rng.uniform(-1, 1, (6, 5)), rng.uniform(-1, 1, 5)
    contract_fixture(ref, "accumulate_plus", "A_i += B_i_j C_j", [B, C], rng.uniform(-1, 1, 6))
    contract_fixture(ref, "accumulate_minus_adds", "A_i -= B_i_j C_j", [B, C], rng.uniform(-1, 1, 6))
    contract_fixture(ref, "diagonal", "A_i = B_i_i", [rng.uniform(-1, 1, (5, 5))], np.zeros(5))
    contract_fixture(ref, "trace_broadcast", "A_i = B_j_j", [rng.uniform(-1, 1, (5, 5))], np.zeros(4))

    J = workloads.config2_inputs(E=4, Q=16)
    Ainv, det = ref.batch_matrix_inv_det(J)
    save("cfg2_invdet_64", kind="invdet", A=J, Ainv=Ainv, det=det)
    for m in (1, 2):
        A = np.eye(m) + 0.1 * rng.uniform(-1, 1, (16, m, m))
        Ainv, det = ref.batch_matrix_inv_det(A)
        save("invdet_%dx%d" % (m, m), kind="invdet", A=A, Ainv=Ainv, det=det)

    M = np.array([0, 1, 2, 3, 4, 5, 1, 3], dtype=np.int32)
    src, vals = rng.uniform(-1, 1, 6), rng.uniform(-1, 1, 8)
    save("scatter_gather_8_to_6", kind="gather", M=M, domain=6, src=src, vals=vals, scattered=ref.scatter(src, M),
         gathered=ref.sum_gather(vals, M, 6))


if __name__ == "__main__":
    main()
