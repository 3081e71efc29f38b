"""Seeded random kernels and random multi-kernel chains on the GPU against the checker: exercises the generator's
scheduling decisions (tiles, phases shared by independent kernels, register forwarding, LDS tiles, views, transient
elision, prefetch, reduction and counted-loop paths) on shapes nobody hand-picked."""
import numpy as np
import pytest

from gpu_helpers import rel_err, to_tensor

pytestmark = pytest.mark.gpu
TOL = 1e-12
LETTERS = "abcdfghijklmnopqrstuvwxyz"


def random_single_kernel(rng):
    n_out = int(rng.integers(1, 4))
    n_con = int(rng.integers(0, 3))
    names = list(rng.choice(list(LETTERS), size=n_out + n_con, replace=False))
    out_idx, con_idx = names[:n_out], names[n_out:]
    extent = {n: int(rng.integers(1, 6)) for n in names}
    extent[out_idx[0]] = int(rng.integers(1, 70))
    if con_idx and rng.random() < 0.2:
        extent[con_idx[0]] = int(rng.integers(600, 3000))      # long contraction: counted-loop / reduction paths
    n_in = int(rng.integers(1, 4))
    ins = []
    for v in range(n_in):
        k = int(rng.integers(1, len(names) + 1))
        ins.append(list(rng.choice(names, size=k, replace=False)))
    for c in con_idx:                                          # every contraction index must appear somewhere
        if not any(c in i for i in ins):
            ins[int(rng.integers(0, n_in))].append(c)
    op = rng.choice(["=", "=", "+=", "-="])
    kernel = "O_" + "_".join(out_idx) + " " + op + " " + " ".join("I%d_%s" % (v, "_".join(i)) for v, i in enumerate(ins))
    shapes = [tuple(extent[n] for n in i) for i in ins]
    return kernel, tuple(extent[n] for n in out_idx), shapes, op


@pytest.mark.parametrize("seed", range(40))
def test_random_single_kernels(at, engine, checker, seed):
    rng = np.random.default_rng(1000 + seed)
    kernel, out_shape, shapes, op = random_single_kernel(rng)
    print(kernel, out_shape, shapes, flush=True)
    ins = [rng.uniform(-1, 1, s) for s in shapes]
    init = rng.uniform(-1, 1, out_shape)
    out = to_tensor(at, init)
    engine(kernel, out, *[to_tensor(at, a) for a in ins])
    out.MoveFromGPU()
    expected = init.copy()
    checker.contract(kernel.replace("-=", "+="), expected, *ins)
    if op == "-=":
        expected = init - (expected - init)
    assert rel_err(out.data, expected) <= TOL


def random_chain(rng):
    """A chain of kernels that all carry the element index e first; later kernels read earlier results."""
    E = int(rng.integers(1, 50))
    pool = {}            # name -> (index names, array or None for computed)
    extent = {"e": E}

    def ext(n):
        if n not in extent:
            extent[n] = int(rng.integers(1, 6))
        return extent[n]

    kernels = []
    n_kernels = int(rng.integers(2, 7))
    produced = []
    for k in range(n_kernels):
        n_mid = int(rng.integers(0, 3))
        mids = list(rng.choice(list("ijklmn"), size=n_mid, replace=False))
        cons = list(rng.choice(list("pqrs"), size=int(rng.integers(0, 3)), replace=False))
        out_name = "R%d" % k
        if produced and rng.random() < 0.15:
            out_name = produced[int(rng.integers(0, len(produced)))]      # overwrite / accumulate into an earlier result
            out_idx = pool[out_name][0]
            mids = [n for n in out_idx if n != "e"]
        else:
            out_idx = ["e"] + mids
        ins = []
        if produced and rng.random() < 0.8:
            src = produced[int(rng.integers(0, len(produced)))]
            if src != out_name:
                ins.append(src)
        n_fresh = int(rng.integers(1, 3)) if not ins else int(rng.integers(0, 3))
        for f in range(n_fresh):
            name = "F%d%d" % (k, f)
            avail = ["e"] + mids + cons
            idx = list(rng.choice(avail, size=int(rng.integers(1, len(avail) + 1)), replace=False))
            pool[name] = (idx, None)
            ins.append(name)
        used = set(n for i in ins for n in pool[i][0])
        missing = [c for c in cons if c not in used]
        if missing:
            name = "F%dx" % k
            pool[name] = (["e"] + missing if rng.random() < 0.5 else missing, None)
            ins.append(name)
        # indices of read results that the output does not carry become contraction indices automatically
        op = "=" if out_name not in produced else rng.choice(["=", "+="])
        if out_name not in pool:
            pool[out_name] = (out_idx, None)
            produced.append(out_name)
        kernels.append((out_name, op, ins))
    shapes = {n: tuple(ext(i) for i in idx) for n, (idx, _) in pool.items()}
    strings = []
    for out_name, op, ins in kernels:
        spell = lambda n: n + "_" + "_".join(pool[n][0])
        strings.append((spell(out_name) + " " + op + " " + " ".join(spell(i) for i in ins), out_name, ins))
    return strings, shapes, produced


@pytest.mark.parametrize("seed", range(40))
def test_random_chains(at, engine, checker, seed):
    run_random_chain(at, engine, checker, 5000 + seed)


@pytest.mark.parametrize("seed", range(40))
def test_random_chains_with_every_possible_kernel_reordered(at, engine, checker, monkeypatch, seed):
    # kernels of the chain with three or more operands are split into steps whenever that is cheaper at all
    # (thresholds off): generator-owned partial results next to the user's intermediates in one fused launch
    monkeypatch.setenv("ACRO_HIP_FACTORISE", "2")
    run_random_chain(at, engine, checker, 7000 + seed)


def forward_chain(rng):
    """Random chain whose kernels all enumerate the same work items (the batch index e plus up to two more indices):
    later kernels read earlier results entry by entry, under their own or other small index names, also twice and
    also as the operand of a contraction, so the generator can apply them in the producer's registers.  Now and then
    a batched matrix inverse or determinant of an earlier result joins the chain.
    Returns (steps, shapes, produced names, names holding matrices); a step is (kernel string | "inv" | "det", out, ins)."""
    items = ["e"] + list(rng.choice(["u", "v"], size=int(rng.integers(0, 3)), replace=False))
    extent = {"e": int(rng.integers(1, 40)), "u": int(rng.integers(1, 7)), "v": int(rng.integers(1, 7))}
    m = int(rng.integers(1, 4))                    # every small index has this extent, so that any may rename any
    small = list("abcdfg")
    for n in small:
        extent[n] = m
    shapes, produced, steps, mats = {}, [], [], set()
    dims = {}                                       # produced name -> number of small dimensions
    for k in range(int(rng.integers(2, 6))):
        out = "R%d" % k
        if rng.random() < 0.3:
            # a well-conditioned matrix per work item (the fresh input is filled with identity + noise), copied by a
            # kernel of the chain, then inverted and / or its determinant taken
            idx = items + list(rng.choice(small, size=2, replace=False))
            shapes["M%d" % k] = shapes[out] = tuple(extent[i] for i in idx)
            mats.add("M%d" % k)
            dims[out] = 2
            steps.append((out + "_" + "_".join(idx) + " = M%d_" % k + "_".join(idx), out, ["M%d" % k]))
            produced.append(out)
            which = int(rng.integers(0, 3))
            if which != 1:
                shapes[out + "i"], dims[out + "i"] = shapes[out], 2
                steps.append(("inv", out + "i", [out]))
                produced.append(out + "i")
            if which != 0:
                shapes[out + "d"], dims[out + "d"] = shapes[out][:-2], 0
                steps.append(("det", out + "d", [out]))
                produced.append(out + "d")
            continue
        out_small = list(rng.choice(small, size=int(rng.integers(0, 3)), replace=False))
        ins, names = [], []
        for p in (rng.choice(produced, size=min(len(produced), int(rng.integers(1, 3))), replace=False) if produced else []):
            for _ in range(int(rng.integers(1, 3))):
                idx = items + list(rng.choice(small, size=dims[p], replace=False))
                ins.append(str(p) + "_" + "_".join(idx))
                names.append(str(p))
        for f in range(int(rng.integers(1, 3))):
            name = "F%d%d" % (k, f)
            idx = list(rng.choice(items + small, size=int(rng.integers(1, 4)), replace=False))
            shapes[name] = tuple(extent[i] for i in idx)
            ins.append(name + "_" + "_".join(idx))
            names.append(name)
        op = "=" if rng.random() < 0.8 else "+="
        shapes[out] = tuple(extent[i] for i in items + out_small)
        dims[out] = len(out_small)
        steps.append((out + "_" + "_".join(items + out_small) + " " + op + " " + " ".join(ins), out, names))
        produced.append(out)
    return steps, shapes, produced, mats


def run_random_chain(at, engine, checker, seed):
    rng = np.random.default_rng(seed)
    strings, shapes, produced = random_chain(rng)
    for s, _, _ in strings:
        print(s, flush=True)
    print(shapes, flush=True)
    arrays = {n: rng.uniform(-1, 1, shp) for n, shp in shapes.items()}
    transient = [n for n in produced[:-1] if rng.random() < 0.5]
    tensors = {n: to_tensor(at, a) for n, a in arrays.items()}
    for n in transient:
        tensors[n].SetTransient(True)
    engine.BeginMultiKernelLaunch()
    for s, out, ins in strings:
        engine(s, tensors[out], *[tensors[i] for i in ins])
    engine.EndMultiKernelLaunch()
    expected = {n: a.copy() for n, a in arrays.items()}
    for s, out, ins in strings:
        checker.contract(s, expected[out], *[expected[i] for i in ins])
    for n in produced:
        if n in transient:
            continue
        tensors[n].MoveFromGPU()
        assert rel_err(tensors[n].data, expected[n]) <= TOL, n


def run_forward_chain(at, engine, checker, seed):
    rng = np.random.default_rng(seed)
    steps, shapes, produced, mats = forward_chain(rng)
    for s in steps:
        print(s, flush=True)
    arrays = {n: np.eye(shp[-1]) + 0.2 * rng.uniform(-1, 1, shp) if n in mats else rng.uniform(-1, 1, shp)
              for n, shp in shapes.items()}
    transient = [n for n in produced[:-1] if rng.random() < 0.5]
    tensors = {n: to_tensor(at, a) for n, a in arrays.items()}
    for n in transient:
        tensors[n].SetTransient(True)
    engine.BeginMultiKernelLaunch()
    for s, out, ins in steps:
        if s == "inv":
            engine.BatchMatrixInverse(tensors[out], tensors[ins[0]])
        elif s == "det":
            engine.BatchMatrixDet(tensors[out], tensors[ins[0]])
        else:
            engine(s, tensors[out], *[tensors[i] for i in ins])
    engine.EndMultiKernelLaunch()
    expected = {n: a.copy() for n, a in arrays.items()}
    for s, out, ins in steps:
        if s == "inv":
            expected[out][...] = checker.batch_matrix_inv_det(expected[ins[0]])[0]
        elif s == "det":
            expected[out][...] = checker.batch_matrix_inv_det(expected[ins[0]])[1]
        else:
            checker.contract(s, expected[out], *[expected[i] for i in ins])
    for n in produced:
        if n in transient:
            continue
        tensors[n].MoveFromGPU()
        assert rel_err(tensors[n].data, expected[n]) <= 10 * TOL, n     # products of up to six factors
    return engine.GetLastImplementation()


@pytest.mark.parametrize("seed", range(45))
def test_random_chains_over_the_same_work_items(at, engine, checker, seed):
    # kernels applied in the registers of their producers, matrix inverses and determinants among them; seed 41 is a
    # capture that a matrix operation without reader splits into three launches while a transient result of the
    # first is an operand of the last
    run_forward_chain(at, engine, checker, 90000 + seed)
