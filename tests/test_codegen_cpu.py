"""The code generator and the hipRTC compile step run without a device: generate, compile for gfx950 and inspect
the source of kernels for the five baseline configurations and for the schedule's corner cases."""
import numpy as np
import pytest

import acrotensor_amd as at
from acrotensor_amd import workloads


@pytest.fixture(scope="module")
def TE():
    return at.TensorEngine("HIP")


def chain_source(TE, wl, transient):
    tensors = workloads.bind_to_engine(wl, at, transient=transient)
    TE.BeginMultiKernelLaunch()
    for k, out, ins in wl.kernels:
        TE(k, tensors[out], *[tensors[n] for n in ins])
    return TE.EndMultiKernelLaunchGetImplementation()


def test_single_contraction_source(TE):
    A, C, B = at.Tensor(64, 9), at.Tensor(64, 9, 5), at.Tensor(5)
    src = TE.GetImplementation("A_e_i = C_e_i_j B_j", A, C, B)
    assert 'extern "C" __global__' in src and "__launch_bounds__" in src
    assert "A_e_i = C_e_i_j B_j" in src                      # the kernel string is quoted in a comment
    assert "batch index e extent 64" in src
    assert "address_space(4)" in src and "B<-scalar" in src   # the small invariant operand is read with scalar loads


def test_mass_apply_chain_keeps_intermediates_on_chip(TE):
    src = chain_source(TE, workloads.config4(E=64), transient=True)
    assert src.count("__syncthreads()") == 5                  # 7 kernels, one applied in registers: 6 phases
    assert "in-register after previous" in src
    assert "T1->lds" in src and "V2->lds" in src and "Y->global" in src
    assert "T3<-registers" in src and "D<-global" in src
    # no store of a transient intermediate to device memory: only Y (parameter of the last kernel) is written
    stores = [l.strip() for l in src.splitlines() if "] = r" in l or "__builtin_nontemporal_store" in l]
    stores = [l for l in stores if not l.startswith("lds[")]
    assert stores and all("T9[" in l for l in stores)


def test_mass_apply_chain_stores_everything_by_default(TE):
    src = chain_source(TE, workloads.config4(E=64), transient=False)
    for name in ("T1", "T2", "U", "V1", "V2"):
        assert name + "->lds+global" in src
        # ... and they reach device memory from their LDS tiles, whole lines at a time, after the phase's barrier
        assert "// %s: LDS tiles -> device memory" % name in src
    assert "T3->global" in src and "// T3: LDS tiles" not in src     # applied in registers: the lanes store it


def test_mass_assembly_is_evaluated_as_a_chain_of_small_contractions(TE):
    wl = workloads.config3(E=16)
    tensors = workloads.bind_to_engine(wl, at)
    k, out, ins = wl.kernels[0]
    src = TE.GetImplementation(k, tensors[out], *[tensors[n] for n in ins])
    # one index is summed per step; the two partial results are tensors of the generator's own that live in LDS
    assert src.count("contraction=4 unrolled") == 3 and "contraction=64" not in src
    assert "_F1->lds\n" in src and "_F2->lds\n" in src and "_F2<-lds" in src
    # a launch that writes far more than it reads and whose lanes would store pieces of 72 bytes: the result leaves
    # through an LDS tile, whole lines per store instruction
    assert "M->lds+global" in src and "// M: LDS tiles -> device memory" in src
    assert src.count("__syncthreads()") == 3
    # kernel parameters are the user's tensors only: M, B, W
    signature = [l for l in src.splitlines() if "__global__" in l][0]
    assert signature.count("double *") == 3
    # the last step keeps the slowest output indices in the lane's tile, so lanes follow the fast dimensions
    assert "lanes(j,k,m,n)=81 tile(i,l)=9" in src
    # as written: 729 * 64 * 6 multiplications per element; the chain needs about 4 800 multiply-adds
    assert src.count("*") < 1500


def test_mass_assembly_without_reordering_shares_partial_sums_inside_the_lane(TE, monkeypatch):
    monkeypatch.setenv("ACRO_HIP_FACTORISE", "-1")
    wl = workloads.config3(E=17)
    tensors = workloads.bind_to_engine(wl, at)
    k, out, ins = wl.kernels[0]
    src = TE.GetImplementation(k, tensors[out], *[tensors[n] for n in ins])
    assert ")=9 contraction=64 unrolled" in src           # a 3x3 tile of outputs per lane
    # as written the kernel has 729 * 64 * 6 multiplications per element; hoisting leaves a small fraction
    assert src.count("*") < 81 * 400


def test_small_or_barely_cheaper_kernels_are_not_reordered(TE):
    # geometric-factor setup (reference unittest/kernel/test_TensorEngine.cpp:543-590): summing j first would save
    # a third of the multiplications, which one lane's shared partial sums already do
    D, W, C, Jdet, Jinv = at.Tensor(10, 3, 3, 5, 5, 5), at.Tensor(5, 5, 5), at.Tensor(10, 5, 5, 5), at.Tensor(10, 5, 5, 5), at.Tensor(10, 5, 5, 5, 3, 3)
    src = TE.GetImplementation("D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j",
                               D, W, C, Jdet, Jinv, Jinv)
    assert "_F1" not in src and src.count("__syncthreads()") == 0


def test_stiffness_assembly_sums_one_direction_early(TE):
    # 3D stiffness assembly (reference unittest/kernel/test_TensorEngine.cpp:437-496): 1 125 terms of 4 factors per
    # output as written; the k3 sum is taken first, the remaining directions would not fit in LDS
    S, B1, B2, B3, D = at.Tensor(10, 5, 5, 5, 5, 5, 5), at.Tensor(5, 5, 5, 3, 3), at.Tensor(5, 5, 5, 3, 3), at.Tensor(5, 5, 5, 3, 3), at.Tensor(10, 5, 5, 5, 3, 3)
    src = TE.GetImplementation("S_e_i1_i2_i3_j1_j2_j3 = B1_i1_j1_k1_m_n B2_i2_j2_k2_m_n B3_i3_j3_k3_m_n D_e_k1_k2_k3_m_n",
                               S, B1, B2, B3, D)
    assert "_F1->lds\n" in src and "_F1<-lds" in src and "S->global" in src


def test_split_contraction_with_few_outputs_gives_a_lane_whole_slices(TE, monkeypatch):
    S, A, B = at.Tensor(3, 3), at.Tensor(1 << 18, 3, 3), at.Tensor(1 << 18)
    src = TE.GetImplementation("S_i_j = A_n_i_j B_n", S, A, B)
    assert "a lane owns whole slices" in src and "split over 256 workgroups" in src
    assert src.count("double acc") == 9 and src.count("T2[ob1") == 1      # B is loaded once per slice, not per output
    assert src.count("__global__") == 2 and "atomic" not in src            # second kernel adds the partials
    # outputs that are not the fastest dimension of the big operand: 64 adjacent lanes walk along each row, four
    # rows per workgroup, and the grid covers groups of rows as well as shares of the contraction
    S2, A2 = at.Tensor(40), at.Tensor(40, 1 << 14)
    src = TE.GetImplementation("S_i = A_i_n B_n", S2, A2, at.Tensor(1 << 14))
    assert "four outputs per workgroup, 64 adjacent lanes along each" in src and "blockIdx.x % 10" in src
    # at most four such outputs: all of them in every workgroup
    src = TE.GetImplementation("S_i = A_i_n B_n", at.Tensor(4), at.Tensor(4, 1 << 14), at.Tensor(1 << 14))
    assert "slices on adjacent lanes" in src
    # many outputs that are the fastest dimension: one lane per (slice, output)
    src = TE.GetImplementation("S_i = A_n_i B_n", at.Tensor(40), at.Tensor(1 << 14, 40), at.Tensor(1 << 14))
    assert "output entries on adjacent lanes" in src
    monkeypatch.setenv("ACRO_HIP_ONE_PASS", "1")
    src = TE.GetImplementation("S_i_j = A_n_i_j B_n", S, at.Tensor((1 << 18) + 1, 3, 3), at.Tensor((1 << 18) + 1))
    assert src.count("__global__") == 1 and "__hip_atomic_fetch_add" in src


def test_many_outputs_summed_over_the_batch_take_the_gram_schedule(TE):
    src = TE.GetImplementation("A_i_j = B_e_i C_e_j", at.Tensor(64, 64), at.Tensor(100000, 64), at.Tensor(100000, 64))
    assert "Gram schedule on the FP64 matrix cores: 64 x 64 outputs, sums over 100000 rows" in src and src.count("__global__") == 2
    assert "acc[ti][tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(bv[u][ti], cv[u][tj], acc[ti][tj], 0, 0, 0);" in src and "atomic" not in src
    # rows of the range past its end and outputs past the last read as zero; the result stored as J x I; a weight per row
    src = TE.GetImplementation("A_j_i -= B_e_q_i C_e_q_j W_e_q", at.Tensor(50, 40), at.Tensor(1001, 3, 40), at.Tensor(1001, 3, 50), at.Tensor(1001, 3))
    assert "40 x 50 outputs (stored transposed), sums over 3003 rows" in src and "(inRange && 16 * ti + r < 40) ? b[16 * ti] : 0.0;" in src
    assert "sums[j * 40 + i]" in src and "bq[u][ti] *= w;" in src and "result[0 + o] - t;" in src
    # up to 128 outputs: the reduction schedule; more than 16 blocks of 16 x 16: neither
    assert "reduction schedule" in TE.GetImplementation("A_i_j = B_e_i C_e_j", at.Tensor(8, 8), at.Tensor(100000, 8), at.Tensor(100000, 8))
    assert "Gram schedule" not in TE.GetImplementation("A_i_j = B_e_i C_e_j", at.Tensor(80, 80), at.Tensor(100000, 80), at.Tensor(100000, 80))
    # the range must lead both operands
    assert "Gram schedule" not in TE.GetImplementation("A_i_j = B_i_e C_e_j", at.Tensor(64, 64), at.Tensor(64, 100000), at.Tensor(100000, 64))


def test_entry_last_layouts_number_the_items_with_the_entry_fastest(TE):
    src = TE.GetImplementation("A_i_e = B_i_e C_i_e", at.Tensor(16, 100000), at.Tensor(16, 100000), at.Tensor(16, 100000))
    assert "64 per workgroup of 256 lanes, numbered with the entry fastest" in src and "const int b = w & 63;" in src and "const int r_ = w / 64;" in src
    # one tensor with the entry first, or a small batch: the usual numbering
    assert "entry fastest" not in TE.GetImplementation("A_i_e = B_e_i C_i_e", at.Tensor(16, 100000), at.Tensor(100000, 16), at.Tensor(16, 100000))
    assert "entry fastest" not in TE.GetImplementation("A_i_e = B_i_e C_i_e", at.Tensor(16, 1000), at.Tensor(16, 1000), at.Tensor(16, 1000))


def test_long_contraction_uses_counted_loops(TE):
    wl = workloads.config1(n=4096)
    tensors = workloads.bind_to_engine(wl, at)
    k, out, ins = wl.kernels[0]
    src = TE.GetImplementation(k, tensors[out], *[tensors[n] for n in ins])
    assert "looped" in src or "split" in src


def test_diffusion_chain_resolves_slices_of_one_tensor_and_fuses(TE):
    # U0, U1, U2 are written under their own names and read back through U (and Z the other way round): the
    # generator resolves the views of one tensor exactly and keeps all of it on chip
    src = chain_source(TE, workloads.config5(E=2, Q=5, P=4), transient=True)
    assert src.count("__global__") == 1 and "not fused" not in src
    assert "U<-lds" in src and "Z0<-lds" in src and "Z2<-lds" in src
    assert "U0->lds\n" in src and "Z->lds\n" in src            # transient: no store to device memory
    # Y is accumulated by three kernels in registers; only the last one stores it
    assert src.count("Y->\n") == 2 and src.count("Y->global") == 1
    # independent kernels share a phase: 18 kernels run in 7 barrier-separated phases
    assert src.count("__syncthreads()") == 6


def test_diffusion_chain_batching_follows_the_contractions_not_the_pointwise_kernel(TE):
    # Q=6, P=5: the pointwise kernel Z = D U has 216 lanes, the 17 contractions 25 - 36.  One element per workgroup
    # must not turn X into a scalar operand (6 busy lanes for T1 instead of 25) ...
    src = chain_source(TE, workloads.config5(E=64, Q=6, P=5), transient=True)
    assert "T1g_e_q_j_k = G_q_i X_e_i_j_k : lanes(j,k)=25" in src and "G<-scalar X<-global" in src
    # ... and with Q=5, P=4 (125 lanes against 16 - 25) several elements share a workgroup although the pointwise
    # kernel then needs more than one pass over its items
    src = chain_source(TE, workloads.config5(E=64, Q=5, P=4), transient=True)
    header = src.splitlines()[1]
    per_group = int(header.split(",")[1].split()[0])
    assert per_group >= 2 and "256 lanes" in header
    assert src.count("__syncthreads()") == 6


def test_small_invariant_operand_read_by_rows_is_staged_in_lds(TE):
    # lane i walks along row i of B: from device memory every load instruction would touch 64 lines; each workgroup
    # copies B to LDS once (row stride 65, so that the lanes fall into different banks) and serves 16 entries
    src = TE.GetImplementation("A_e_i = B_i_j X_e_k_j W_e_k", at.Tensor(1000, 64), at.Tensor(64, 64), at.Tensor(1000, 2, 64), at.Tensor(1000, 2))
    assert "B<-lds" in src and "// B: device memory -> LDS, once per workgroup" in src
    assert "a += (r_ / 64) * 65" in src and "16 per workgroup of 256 lanes" in src
    assert src.index("__syncthreads()") < src.index("// A_e_i = B_i_j X_e_k_j W_e_k")
    # a table that the lanes read at unit stride, or one read through scalar loads, is left where it is
    assert "<-lds" not in TE.GetImplementation("A_e_i = B_j_i X_e_j", at.Tensor(1000, 64), at.Tensor(64, 64), at.Tensor(1000, 64))
    assert "B<-scalar" in TE.GetImplementation("A_e_q_j = B_q_i X_e_i_j", at.Tensor(500, 5, 16), at.Tensor(5, 4), at.Tensor(500, 4, 16))


def test_streaming_kernels_with_light_workgroups_take_more_entries(TE, monkeypatch):
    E = 100000
    # 2 entries x (8 + 8 + 64) doubles = 1.3 KB per workgroup: raised to 16 entries in four passes of 256 lanes
    outer = lambda: TE.GetImplementation("A_e_i_j = B_e_i C_e_j", at.Tensor(E, 8, 8), at.Tensor(E, 8), at.Tensor(E, 8))
    assert "16 per workgroup of 256 lanes" in outer() and "w0 < 1024; w0 += 256" in outer()
    assert "32 per workgroup of 256 lanes" in TE.GetImplementation("A_e_i = B_e_i", at.Tensor(E, 16), at.Tensor(E, 16))
    # 3 KB per workgroup and more stay as they are (the old value of += counts), unless an item has four factors or more
    assert "8 per workgroup of 128 lanes" in TE.GetImplementation("A_e_i += B_e_i", at.Tensor(E, 16), at.Tensor(E, 16))
    assert "16 per workgroup of 256 lanes" in TE.GetImplementation("A_e_i = B_e_i C_e_i D_i F_e", at.Tensor(E, 32), at.Tensor(E, 32), at.Tensor(E, 32), at.Tensor(32), at.Tensor(E))
    assert "8 per workgroup of 128 lanes" in TE.GetImplementation("A_e_i = B_e_i C_e_i D_e_i", *[at.Tensor(E, 16)] * 4)
    # one entry of 256 items per workgroup, an item per lane: two entries in two passes
    assert "2 per workgroup of 256 lanes" in TE.GetImplementation("A_e_i_j = B_e_i_j C_i_j", at.Tensor(E, 16, 16), at.Tensor(E, 16, 16), at.Tensor(16, 16))
    # 512 pointwise items per entry: two passes of 256 lanes
    assert "1 per workgroup of 256 lanes" in TE.GetImplementation("A_e_i_j = B_e_i_j C_i_j", at.Tensor(E, 16, 32), at.Tensor(E, 16, 32), at.Tensor(16, 32))
    # few entries: never more than there are
    assert "batch index e extent 9, 8 per workgroup" in TE.GetImplementation("A_e_i_j = B_e_i C_e_j", at.Tensor(9, 8, 8), at.Tensor(9, 8), at.Tensor(9, 8))
    monkeypatch.setenv("ACRO_HIP_LIGHT", "-1")     # (other sizes: the engine keeps what it generated for the sizes above)
    assert "2 per workgroup of 256 lanes" in TE.GetImplementation("A_e_i_j = B_e_i C_e_j", at.Tensor(E + 1, 8, 8), at.Tensor(E + 1, 8), at.Tensor(E + 1, 8))


def test_dense_operator_per_entry_uses_the_operator_schedule(TE, monkeypatch):
    # FP64 matrix cores, 16 entries per wavefront and trip
    src = TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(1000, 64), at.Tensor(64, 64), at.Tensor(1000, 64))
    assert "operator schedule on the FP64 matrix cores: 64 x 64 operator in LDS in operand order, 1000 entries" in src
    assert "__builtin_amdgcn_mfma_f64_16x16x4f64(xs, frag[(t * 16 + step) * 64 + lane], acc[t], 0, 0, 0)" in src
    assert "j = 8 * (step >> 1) + 2 * (l >> 4) + (step & 1);" in src and "a + 4 * r * 64 + 16 * t" in src
    assert "tile * 16 + c < 1000 ? tile * 16 + c : 999" in src and "if (tile * 16 + g + 4 * r >= 1000) continue;" in src
    src = TE.GetImplementation("A_e_i += B_i_j X_e_j", at.Tensor(1024, 32), at.Tensor(32, 24), at.Tensor(1024, 24))
    assert "32 x 24 operator" in src and "padded" not in src and "a[4 * r * 32 + 16 * t] += acc[t][r];" in src and "continue" not in src
    # the operator stored transposed, and two leading indices that number the entries
    src = TE.GetImplementation("A_e_q_i = B_j_i X_e_q_j", at.Tensor(100, 7, 32), at.Tensor(24, 32), at.Tensor(100, 7, 24))
    assert "32 x 24 operator (stored transposed) in LDS in operand order, 700 entries" in src
    assert "T1[0 + j * 32 + row]" in src and "tile * 16 + c < 700" in src
    # sizes that 16 x 4 blocks do not divide: zero rows and columns in LDS, guarded loads and stores; an odd row
    # length means single 8-byte loads of the entries' vectors
    src = TE.GetImplementation("A_e_i1_i2 -= X_e_j1_j2 B_i1_i2_j1_j2", at.Tensor(77, 5, 6), at.Tensor(77, 4, 7), at.Tensor(5, 6, 4, 7))
    assert "30 x 28 operator in LDS in operand order (padded to 32 x 32)" in src
    assert "frag[f] = row < 30 && j < 28 ? T2[0 + row * 28 + j] : 0.0;" in src
    assert "8 * q + 2 * g >= 28 ? double2{0.0, 0.0} :" in src and "if (16 * t + c < 30) mid[(4 * r + g) * 30 + 16 * t + c] = acc[t][r];" in src and "a[i] -= mid[i];" in src
    src = TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(1000, 30), at.Tensor(30, 27), at.Tensor(1000, 27))
    assert "(padded to 32 x 28)" in src and "j = 4 * step + (l >> 4);" in src and "xv[q] = 4 * q + g >= 27 ? 0.0 : x[4 * q];" in src
    # pointwise factors: per entry, per output and per row on the result, per element and per column on the vectors
    # (an operator below 16 x 16 on its own keeps the generic schedule; the switch brings it here, as a group would)
    factors = ("A_e_i -= B_i_j X_e_j W_e D_e_j R_i F_e_i C_j", at.Tensor(1000, 10), at.Tensor(10, 12), at.Tensor(1000, 12),
               at.Tensor(1000), at.Tensor(1000, 12), at.Tensor(10), at.Tensor(1000, 10), at.Tensor(12))
    assert "operator schedule" not in TE.GetImplementation(*factors)
    monkeypatch.setenv("ACRO_HIP_OPERATOR_SMALL", "-1")
    src = at.TensorEngine("HIP").GetImplementation(*factors)
    monkeypatch.delenv("ACRO_HIP_OPERATOR_SMALL")
    assert "operator schedule on the FP64 matrix cores: 10 x 12 operator" in src and "const double se = T3[0 + en];" in src
    # (10 rows: the results of a trip's 16 entries are collected in LDS in memory order and leave as one contiguous range)
    assert "mid[(4 * r + g) * 10 + 16 * t + c] = acc[t][r] * se * T6[0 + en * 10 + 16 * t + c] * T5[0 + 16 * t + c];" in src
    assert "results written out through LDS" in src and "for (int i = lane; i < count; i += 64)" in src and "a[i] -= mid[i];" in src
    assert "const acro_pair f = *reinterpret_cast<const acro_pair *>(T4 + 0 + ex * 12 + 2 * g + 8 * q);" in src and "const double *f = T7 + 0 + 2 * g + 8 * q;" in src
    # the entries as the fastest dimension: the operator becomes the instruction's first operand
    src = TE.GetImplementation("A_i_e -= B_i_j X_j_e W_e", at.Tensor(30, 1002), at.Tensor(30, 27), at.Tensor(27, 1002), at.Tensor(1002))
    assert "matrix cores, entries fastest: 30 x 27 operator in LDS in operand order (padded to 32 x 28), 1002 entries, 32 per wavefront" in src
    assert "acc1[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step].y, acc1[t], 0, 0, 0);" in src and "const long ex = e < 1002 ? e : 1000;" in src
    src = TE.GetImplementation("A_i_e = B_i_j X_j_e", at.Tensor(64, 1001), at.Tensor(64, 64), at.Tensor(64, 1001))
    assert "1001 entries, 16 per wavefront and trip" in src and "__builtin_nontemporal_store(v, a);" in src and "acc1" not in src
    assert "operator schedule" not in TE.GetImplementation("A_i_e = B_i_j X_j_e", at.Tensor(16, 3000), at.Tensor(16, 16), at.Tensor(16, 3000))
    # an operator too large for LDS: blocks of rows, a launch each
    src = TE.GetImplementation("G_e_d_q = D_d_q_i X_e_i", at.Tensor(1000, 3, 64), at.Tensor(3, 64, 64), at.Tensor(1000, 64))
    assert "rows 0 - 127 of the 192 x 64 operator" in src and "rows 128 - 191 of the 192 x 64 operator" in src and src.count("__global__") == 2
    assert "frag[f] = T1[0 + (row + 128) * 64 + j];" in src and "double *a = T0 + 0 + (tile * 16 + g) * 192 + 128 + c;" in src
    # one shared factor of 4 097 to 8 192 entries and at most 96 columns goes to the operator schedule where that applies,
    # and stays a tiled product where it does not (vectors stored entries-fastest) or above those sizes
    src = TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(1003, 125), at.Tensor(125, 64), at.Tensor(1003, 64))
    assert "rows 0 - 124 of the 125 x 64 operator in LDS in operand order (padded to 128 x 64)" in src and src.count("__global__") == 1
    for shapes in [((1003, 125), (125, 125), (1003, 125)), ((1003, 64), (64, 125), (1003, 125))]:
        assert "tiled product schedule" in TE.GetImplementation("A_e_i = B_i_j X_e_j", *[at.Tensor(*sh) for sh in shapes])
    assert "tiled product schedule" in TE.GetImplementation("A_e_i = B_i_j X_j_e", at.Tensor(1003, 125), at.Tensor(125, 64), at.Tensor(64, 1003))
    # the operator's dimensions in any order: its copy in LDS is filled through their strides
    src = TE.GetImplementation("J_e_q_n_m = G_q_i_n X_e_i_m", at.Tensor(501, 27, 3, 3), at.Tensor(27, 27, 3), at.Tensor(501, 27, 3))
    assert "81 x 27 operator (dimensions in another order)" in src and "3 components per vector element" in src
    assert "T1[0 + (row % 3) * 1 + ((row / 3) % 27) * 81 + (j % 27) * 3]" in src
    # components between the result's row indices: put into memory order while a trip's results are collected in LDS
    src = TE.GetImplementation("J_e_q_m_n = X_e_i_m G_q_i_n", at.Tensor(501, 27, 3, 3), at.Tensor(501, 27, 3), at.Tensor(27, 27, 3))
    assert "81 x 27 operator (dimensions in another order)" in src and "3 components per vector element, results written out through LDS" in src
    assert "mid[(4 * r + g) * 243 + ((16 * t + c) % 3) * 1 + (((16 * t + c) / 3) % 27) * 9 + (k % 3) * 3] = acc[k][t][r];" in src
    # (operators applied in blocks of rows store from the registers)
    src = TE.GetImplementation("J_e_q_m_n = X_e_i_m G_q_i_n", at.Tensor(501, 64, 3, 3), at.Tensor(501, 64, 3), at.Tensor(64, 64, 3))
    assert "rows 128 - 191 of the 192 x 64 operator (dimensions in another order)" in src and src.count("__global__") == 2
    assert "a[((16 * t + c + 128) % 3) * 1 + (((16 * t + c + 128) / 3) % 64) * 9 + (k % 3) * 3] = acc[k][t][r];" in src
    # the switch for a kernel that the compiler can only fit into the registers with spills
    assert src.count('#ifdef ACRO_KEEP_OPERATOR_IN_LDS\n        __asm__ volatile("" ::: "memory");\n#endif\n') == 2
    # very long vectors or very many rows would not fit a lane's registers: not this schedule
    assert "operator schedule" not in TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(900, 5), at.Tensor(5, 818), at.Tensor(900, 818))
    assert "operator schedule" not in TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(900, 300), at.Tensor(300, 12), at.Tensor(900, 12))
    # not this schedule: few rows of short vectors (a register tile with scalar operands serves them), third operand
    for kernel, shapes in (("A_e_i = B_i_j X_e_j", [(500, 4), (4, 8), (500, 8)]),
                           ("A_e_i = B_i_j X_e_k_j W_e_k", [(500, 64), (64, 64), (500, 2, 64), (500, 2)])):
        tensors = [at.Tensor(*shp) for shp in shapes]
        assert "operator schedule" not in TE.GetImplementation(kernel, *tensors)
    # two to four rows applied to vectors of 16 values and more (a gradient at a point) do take it
    for rows, cols in ((4, 64), (3, 32), (2, 16)):
        src = TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(500, rows), at.Tensor(rows, cols), at.Tensor(500, cols))
        assert "operator schedule on the FP64 matrix cores: %d x %d operator" % (rows, cols) in src
    # without the matrix cores: a lane keeps its row for four entries, whose vectors come through scalar loads
    monkeypatch.setenv("ACRO_HIP_OPERATOR_MFMA", "-1")
    src = TE.GetImplementation("A_e_i = B_i_j X_e_j", at.Tensor(1000, 60), at.Tensor(60, 60), at.Tensor(1000, 60))
    assert "operator schedule: 60 x 60 operator in LDS (row stride 61), 56 entries per workgroup of 512 lanes" in src
    assert "__builtin_amdgcn_readfirstlane" in src and "acro_scalar_ptr x" in src and src.count("+= b * x[") == 4
    src = TE.GetImplementation("A_e_i1_i2 -= X_e_j1_j2 B_i1_i2_j1_j2", at.Tensor(78, 5, 6), at.Tensor(78, 4, 7), at.Tensor(5, 6, 4, 7))
    assert "operator schedule: 30 x 28 operator" in src and "] -= s3;" in src
    assert "operator schedule" not in TE.GetImplementation("A_e_i = B_j_i X_e_j", at.Tensor(500, 64), at.Tensor(64, 64), at.Tensor(500, 64))


def test_tile_choice_follows_how_the_lanes_reach_device_memory(TE, monkeypatch):
    # one lane per matrix product would read 128-byte pieces 128 bytes apart; tiny entries get one output per lane, from
    # tiles in LDS; entries of whole lines with fewer than 16 outputs are read as well straight from device memory
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 4, 4), at.Tensor(4096, 4, 4), at.Tensor(4096, 4, 4))
    assert "lanes(i,k)=16 tile()=1" in src and "operands staged in LDS" in src and "32 per workgroup of 256 lanes" in src
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 2, 2), at.Tensor(4096, 2, 8), at.Tensor(4096, 8, 2))
    assert "lanes(i,k)=4 tile()=1" in src and "operands staged in LDS" not in src
    # one lane per entry would read 512-byte rows 512 bytes apart and overflow the vector cache: one lane per row
    src = TE.GetImplementation("A_e_i = B_e_i_j C_e_j", at.Tensor(4096, 8), at.Tensor(4096, 8, 8), at.Tensor(4096, 8))
    assert "lanes(i)=8 tile()=1" in src
    # 8 x 8 products: operands copied to LDS first, a 2 x 2 block of outputs per lane (the output indices split in two)
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 8, 8), at.Tensor(4096, 8, 8), at.Tensor(4096, 8, 8))
    assert "operands staged in LDS" in src and "lanes(ihi,khi)=16 tile(ilo,klo)=4" in src
    # 11 x 11: no blocks, one output per lane and some thousand outputs per workgroup; 3 x 3 likewise with some 500
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 11, 11), at.Tensor(4096, 11, 11), at.Tensor(4096, 11, 11))
    assert "8 per workgroup of 256 lanes" in src and "lanes(i,k)=121 tile()=1" in src
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 3, 3), at.Tensor(4096, 3, 3), at.Tensor(4096, 3, 3))
    assert "56 per workgroup of 256 lanes" in src and "operands staged in LDS" in src and "lanes(i,k)=9 tile()=1" in src
    # 25 x 25: blocks of five along one index only (125 lane items per entry; both would leave 25); 35 x 35 and 62 x 62:
    # an entry's operands fill most of a workgroup's LDS; 64 x 64 does not fit
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 25, 25), at.Tensor(4096, 25, 25), at.Tensor(4096, 25, 25))
    assert "operands staged in LDS" in src and "lanes(ihi,k)=125 tile(ilo)=5" in src
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 35, 35), at.Tensor(4096, 35, 35), at.Tensor(4096, 35, 35))
    assert "operands staged in LDS" in src and "lanes(ihi,k)=245 tile(ilo)=5" in src and "1 per workgroup of 256 lanes" in src
    # (beyond 36 x 36, and for extents without a divisor 2, 3 or 5, products run on the matrix cores: see the test of
    # the product schedule; this is what the staged schedule does with them when that is switched off)
    monkeypatch.setenv("ACRO_HIP_PRODUCT", "-1")
    src = at.TensorEngine("HIP").GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 62, 62), at.Tensor(4096, 62, 62), at.Tensor(4096, 62, 62))
    assert "operands staged in LDS" in src and "LDS 61504 bytes" in src
    src = at.TensorEngine("HIP").GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 64, 64), at.Tensor(4096, 64, 64), at.Tensor(4096, 64, 64))
    assert "operands staged in LDS" not in src
    monkeypatch.delenv("ACRO_HIP_PRODUCT")
    # second factor transposed: its copy in LDS has the contracted index in front, the copying lanes follow the operand
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_k_j", at.Tensor(4096, 24, 24), at.Tensor(4096, 24, 24), at.Tensor(4096, 24, 24))
    assert "_S2_e_j_khi_klo = C_e_khi_klo_j : lanes(khi,klo,j)=576" in src
    # slices are not whole tensors: their indices stay as they are
    big = at.Tensor(2, 4096, 8, 8)
    src = TE.GetImplementation("A_e_i_k = B_e_i_j C_e_j_k", at.Tensor(4096, 8, 8), at.SliceTensor(big, 1), at.Tensor(4096, 8, 8))
    assert "operands staged in LDS" in src and "ihi" not in src


def test_sums_over_a_long_index_take_the_reduction_schedule_whatever_the_number_of_outputs(TE):
    # a lane per output and workgroup, the summed range dealt out over the workgroups; a finishing workgroup per 256 outputs
    src = TE.GetImplementation("S_i_j = A_e_i_j", at.Tensor(32, 32), at.Tensor(32768, 32, 32))
    assert "reduction schedule: 1024 output entries, contraction of 32768 terms split over 256 workgroups x 1 slices (256 outputs per workgroup, a lane each)" in src
    assert "for (long c = gc; c < 32768; c += 256)" in src
    # (the finishing kernel: 16 lanes per output, a share of the 256 partial sums each, added through LDS in a fixed order)
    assert "const int o = blockIdx.x * 16 + threadIdx.x % 16, part = threadIdx.x / 16;" in src
    assert "for (long g = part; g < 256; g += 16) t += scratch[g * 1024 + o];" in src
    # (many outputs: a lane each)
    src = TE.GetImplementation("S_i_j = A_e_i_j", at.Tensor(128, 128), at.Tensor(4000, 128, 128))
    assert "const int o = blockIdx.x * 256 + threadIdx.x;" in src
    # up to 256 outputs every workgroup has them all; with the summed index fastest a workgroup takes four rows (up to 1 024)
    assert "output entries on adjacent lanes" in TE.GetImplementation("S_i = A_e_i", at.Tensor(200), at.Tensor(50000, 200))
    assert "four outputs per workgroup" in TE.GetImplementation("S_i = A_i_e", at.Tensor(1000), at.Tensor(1000, 50000))
    # ... and beyond, with a finishing workgroup per 256 outputs again
    src = TE.GetImplementation("S_i = A_i_e", at.Tensor(1025), at.Tensor(1025, 50000))
    assert "four outputs per workgroup" in src and "const int o = blockIdx.x * 256 + threadIdx.x;" in src
    # short sums are not reductions
    assert "reduction schedule" not in TE.GetImplementation("S_i = A_e_i", at.Tensor(5000), at.Tensor(2000, 5000))


def scatter_then_mass_apply_source(TE, transient_x):
    wl = workloads.config4(E=27)
    tensors = workloads.bind_to_engine(wl, at, transient=True)
    dofs, nodes = workloads.hex_mesh_dof_map(3, 3, 3, 3)
    M, L = at.IndexMapping(nodes, dofs.size), at.Tensor(nodes)
    M.map[:] = dofs.ravel()
    tensors["X"].SetTransient(transient_x)
    TE.BeginMultiKernelLaunch()
    TE.FlatIndexedScatter(tensors["X"], L, M)
    for k, out, ins in wl.kernels:
        TE(k, tensors[out], *[tensors[n] for n in ins])
    return TE.EndMultiKernelLaunchGetImplementation()


def test_recorded_scatter_with_transient_result_is_read_through_its_map(TE):
    src = scatter_then_mass_apply_source(TE, True)
    assert src.count("__global__") == 1 and "X<-gathered" in src
    assert "const int *__restrict__ G0m, const double *__restrict__ G0s" in src and "G0s[G0m[o_k0v1 + 0]]" in src
    assert "runs on its own" not in src
    # an element vector that has to exist afterwards: the scatter runs, the chain reads what it wrote
    src = scatter_then_mass_apply_source(TE, False)
    assert "runs on its own" in src and "gathered" not in src and "X<-global" in src


def test_views_that_cannot_be_resolved_fall_back(TE):
    # the same parent viewed with the element index in two different positions cannot be fused
    T = at.Tensor(4, 4)
    A, B = at.Tensor(4, 4), at.Tensor(4, 4)
    TE.BeginMultiKernelLaunch()
    TE("T_e_i = A_e_i", T, A)
    TE("B_e_i = T_i_e", B, T)
    src = TE.EndMultiKernelLaunchGetImplementation()
    assert "not fused" in src


def test_rebinding_one_name_to_two_tensors_switches_to_positional_operands(TE):
    A, B1, B2 = at.Tensor(5, 5), at.Tensor(5, 3), at.Tensor(5, 3)
    src = TE.GetImplementation("A_i_j = B_i_k B_j_k", A, B1, B2)
    assert src.count("const double *") >= 2


def test_runtime_compiler_reports_errors_with_the_log():
    import ctypes
    from acrotensor_amd import _capi
    lib = _capi.load()
    size = ctypes.c_size_t(0)
    good = b'extern "C" __global__ void k(double *p) { p[threadIdx.x] = 1.0; }'
    assert lib.acro_hip_compile(b"unit_good", good, ctypes.byref(size)) == 0 and size.value > 0
    bad = b'extern "C" __global__ void k(double *p) { p[threadIdx.x] = undeclared_symbol; }'
    assert lib.acro_hip_compile(b"unit_bad", bad, ctypes.byref(size)) != 0
    message = lib.acro_last_error().decode()
    assert "undeclared_symbol" in message and "unit_bad" in message


def generated_sources(TE):
    """Sources of every schedule the generator has: fused chains with and without stored intermediates, reordered
    kernels, split contractions (both finishes), counted loops, a second grid dimension, positional operands."""
    yield "mass apply, transient", chain_source(TE, workloads.config4(E=66), True)
    yield "mass apply, stored", chain_source(TE, workloads.config4(E=66), False)
    yield "diffusion apply", chain_source(TE, workloads.config5(E=3), True)
    yield "diffusion apply, stored", chain_source(TE, workloads.config5(E=3, Q=5, P=4), False)
    wl = workloads.config3(E=5)
    t = workloads.bind_to_engine(wl, at)
    k, out, ins = wl.kernels[0]
    yield "mass assembly", TE.GetImplementation(k, t[out], *[t[n] for n in ins])
    S, A, B = at.Tensor(3, 3), at.Tensor(70000, 3, 3), at.Tensor(70000)
    yield "split contraction", TE.GetImplementation("S_i_j = A_n_i_j B_n", S, A, B)
    yield "split contraction, += and many outputs", TE.GetImplementation("S_i += A_i_n B_n", at.Tensor(40), at.Tensor(40, 9000), at.Tensor(9000))
    yield "counted loops", TE.GetImplementation("C_e = B_e_j V_j", at.Tensor(300), at.Tensor(300, 700), at.Tensor(700))
    yield "second grid dimension", TE.GetImplementation("A_a_b_c_d_f = B_a_b_c_d_f_k C_k", at.Tensor(12, 11, 10, 9, 5),
                                                        at.Tensor(12, 11, 10, 9, 5, 6), at.Tensor(6))
    yield "stiffness assembly", TE.GetImplementation(
        "S_e_i1_i2_i3_j1_j2_j3 = B1_i1_j1_k1_m_n B2_i2_j2_k2_m_n B3_i3_j3_k3_m_n D_e_k1_k2_k3_m_n",
        at.Tensor(4, 5, 5, 5, 5, 5, 5), at.Tensor(5, 5, 5, 3, 3), at.Tensor(5, 5, 5, 3, 3), at.Tensor(5, 5, 5, 3, 3),
        at.Tensor(4, 5, 5, 5, 3, 3))
    yield "one name, two tensors", TE.GetImplementation("A_m_n = B_m_j B_n_j", at.Tensor(3, 3), at.Tensor(3, 4), at.Tensor(3, 4))
    yield "repeated output index", TE.GetImplementation("A_i_i = B_i", at.Tensor(6, 6), at.Tensor(6))
    yield "operand staged in LDS", TE.GetImplementation("A_e_i = B_i_j X_e_k_j W_e_k", at.Tensor(1000, 64), at.Tensor(64, 64), at.Tensor(1000, 2, 64), at.Tensor(1000, 2))
    yield "operator schedule with pointwise factors", TE.GetImplementation("A_e_i -= B_i_j X_e_j W_e D_e_j R_i F_e_i C_j", at.Tensor(1000, 10), at.Tensor(10, 12),
                                                                         at.Tensor(1000, 12), at.Tensor(1000), at.Tensor(1000, 12), at.Tensor(10), at.Tensor(1000, 10), at.Tensor(12))
    yield "operator schedule, entries fastest", TE.GetImplementation("A_i_e -= B_i_j X_j_e W_e D_j_e R_i F_i_e C_j", at.Tensor(30, 1002), at.Tensor(30, 27),
                                                                   at.Tensor(27, 1002), at.Tensor(1002), at.Tensor(27, 1002), at.Tensor(30), at.Tensor(30, 1002), at.Tensor(27))
    yield "operator schedule, entries fastest, one per lane", TE.GetImplementation("A_i_e = B_j_i X_j_e F_i_e", at.Tensor(64, 1001), at.Tensor(64, 64), at.Tensor(64, 1001), at.Tensor(64, 1001))
    yield "operator schedule, two launches", operator_chain_source(TE, 32, 27, 999, False)
    yield "operator schedule, two operators in one kernel", operator_chain_source(TE, 30, 27, 998)
    yield "operator schedule, two operators in one kernel, 64 000 bytes of LDS", operator_chain_source(TE, 64, 27, 997, False)
    yield "operator schedule with pointwise factors, odd length", TE.GetImplementation("A_e_i = B_i_j X_e_j D_e_j C_j W_e", at.Tensor(1000, 20), at.Tensor(20, 17),
                                                                                     at.Tensor(1000, 17), at.Tensor(1000, 17), at.Tensor(17), at.Tensor(1000))
    yield "operator schedule", TE.GetImplementation("A_e_i1_i2 -= X_e_j1_j2 B_i1_i2_j1_j2", at.Tensor(77, 5, 6), at.Tensor(77, 4, 7), at.Tensor(5, 6, 4, 7))
    yield "operator schedule, no padding", TE.GetImplementation("A_e_i1_i2 -= X_e_j1_j2 B_i1_i2_j1_j2", at.Tensor(77, 8, 6), at.Tensor(77, 4, 10), at.Tensor(8, 6, 4, 10))
    yield "operator schedule, odd row length", TE.GetImplementation("A_e_i = B_j_i X_e_j", at.Tensor(500, 17), at.Tensor(33, 17), at.Tensor(500, 33))
    yield "split contraction, few long rows", TE.GetImplementation("S_i += A_i_n B_n", at.Tensor(6), at.Tensor(6, 9000), at.Tensor(9000))
    yield "transpose through LDS tiles", TE.GetImplementation("A_i_e_j -= B_j_e_i", at.Tensor(100, 3, 70), at.Tensor(70, 3, 100))
    yield "operand read through an index map", scatter_then_mass_apply_source(TE, True)
    yield "contraction shared by lanes", TE.GetImplementation("A_e += B_e_i_j C_j_i", at.Tensor(1000), at.Tensor(1000, 5, 7), at.Tensor(7, 5))
    for transient in (True, False):
        yield "geometric factors from the Jacobians", geometric_factor_source(TE, 7, 4, 3, transient)
    yield "geometric factors, 2 x 2", geometric_factor_source(TE, 7, 3, 2, True)
    yield "entries fastest", TE.GetImplementation("A_i_j_e -= B_i_k_e C_k_j_e", at.Tensor(3, 3, 4099), at.Tensor(3, 3, 4099), at.Tensor(3, 3, 4099))
    yield "Gram matrix over the batch", TE.GetImplementation("A_j_i -= B_e_q_i C_e_q_j W_e_q", at.Tensor(50, 40), at.Tensor(1001, 3, 40), at.Tensor(1001, 3, 50), at.Tensor(1001, 3))
    yield "products of element matrices in 2 x 2 blocks", TE.GetImplementation("A_e_i_j += B_e_i_k C_e_j_k", at.Tensor(100, 12, 10), at.Tensor(100, 12, 9), at.Tensor(100, 10, 9))
    yield "products of tiny element matrices", TE.GetImplementation("A_e_i_j = B_e_i_k C_e_k_j", at.Tensor(1001, 3, 3), at.Tensor(1001, 3, 3), at.Tensor(1001, 3, 3))
    yield "operator schedule, blocks of rows", TE.GetImplementation("G_e_d_q -= D_d_q_i X_e_i W_e", at.Tensor(1001, 3, 65), at.Tensor(3, 65, 64), at.Tensor(1001, 64), at.Tensor(1001))
    yield "operator schedule, results through LDS", TE.GetImplementation("A_e_i += B_j_i X_e_j", at.Tensor(2001, 125), at.Tensor(8, 125), at.Tensor(2001, 8))


GEOMETRIC_FACTORS = {
    3: "D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j",
    2: "D_e_m_n_k1_k2 = W_k1_k2 C_e_k1_k2 Jdet_e_k1_k2 Jinv_e_k1_k2_n_j Jinv_e_k1_k2_m_j",
}


def geometric_factor_source(TE, E, Q, dim, transient):
    """Inverse and determinant of the Jacobians and the contraction that turns them into the geometric factors of the
    diffusion operator (reference unittest/kernel/test_TensorEngine.cpp:498-590), recorded as one launch."""
    pts = (Q,) * dim
    J, Jinv, Jdet = at.Tensor(E, *pts, dim, dim), at.Tensor(E, *pts, dim, dim), at.Tensor(E, *pts)
    W, C, D = at.Tensor(*pts), at.Tensor(E, *pts), at.Tensor(E, dim, dim, *pts)
    Jinv.SetTransient(transient)
    Jdet.SetTransient(transient)
    TE.BeginMultiKernelLaunch()
    TE.BatchMatrixInvDet(Jinv, Jdet, J)
    TE(GEOMETRIC_FACTORS[dim], D, W, C, Jdet, Jinv, Jinv)
    return TE.EndMultiKernelLaunchGetImplementation()


def test_matrix_operations_recorded_in_a_launch_are_fused_with_their_reader(TE):
    src = geometric_factor_source(TE, 64, 10, 3, True)
    assert src.count("__global__") == 1 and "__syncthreads" not in src
    assert "(matrix inverse)" in src and "(determinant)" in src
    # one work item per quadrature point holds the inverse, its determinant and the nine geometric factors
    assert "lanes(k1,k2,k3)=1000 tile(n,j)=9" in src and "lanes(k1,k2,k3)=1000 tile(m,n)=9 contraction=3" in src
    assert "Jdet<-registers Jinv<-registers Jinv<-registers" in src
    assert "Jinv->\n" in src and "Jdet->\n" in src and "D->global" in src      # transient results are never stored
    assert "const double det1 = det0;" in src                                      # the determinant is computed once
    assert src.count("#pragma clang fp contract(off)") == 2 and src.count("#pragma clang fp contract(fast)") == 1
    stored = geometric_factor_source(TE, 64, 10, 3, False)
    assert "Jinv->global" in stored and "Jdet->global" in stored and "Jinv<-registers" in stored


def test_matrix_operation_without_a_reader_in_the_launch_runs_on_its_own(TE):
    J, Jinv, Jdet = at.Tensor(8, 3, 3), at.Tensor(8, 3, 3), at.Tensor(8)
    A, B = at.Tensor(8, 4), at.Tensor(8, 4)
    TE.BeginMultiKernelLaunch()
    TE("A_e_i = B_e_i", A, B)
    TE.BatchMatrixInvDet(Jinv, Jdet, J)
    src = TE.EndMultiKernelLaunchGetImplementation()
    assert src.count("__global__") == 1 and "runs on its own" in src and "matrix inverse" not in src
    # ... and so does one whose result is its own operand
    X, V = at.Tensor(8, 3), at.Tensor(8, 3)
    TE.BeginMultiKernelLaunch()
    TE.BatchMatrixInverse(J, J)
    TE("X_e_i = J_e_i_j V_e_j", X, J, V)
    src = TE.EndMultiKernelLaunchGetImplementation()
    assert "runs on its own" in src and "matrix inverse" not in src


def operator_chain_source(TE, nq, nd, entries=1000, transient=True):
    B, X, D = at.Tensor(nq, nd), at.Tensor(entries, nd), at.Tensor(entries, nq)
    U, Y = at.Tensor(entries, nq), at.Tensor(entries, nd)
    U.SetTransient(transient)
    TE.BeginMultiKernelLaunch()
    TE("U_e_k = B_k_j X_e_j D_e_k", U, B, X, D)
    TE("Y_e_i = B_k_i U_e_k", Y, B, U)
    return TE.EndMultiKernelLaunchGetImplementation()


def test_large_dense_operators_in_a_capture_run_as_one_matrix_core_launch_each(TE):
    # two 64 x 64 operators and the hand-over buffer do not fit LDS together
    src = operator_chain_source(TE, 64, 64, transient=False)
    assert src.count("__global__") == 2 and src.count("operator schedule on the FP64 matrix cores") == 2
    assert "[0] U_e_k = B_k_j X_e_j D_e_k" in src and "[1] Y_e_i = B_k_i U_e_k" in src and "(stored transposed)" in src
    # a transient intermediate never leaves the chip: one kernel, handed over through LDS between the two products
    src = operator_chain_source(TE, 32, 27, 1001)
    assert src.count("__global__") == 1 and "applied to the first result on chip (handed over through 4224 bytes of LDS per wavefront)" in src
    assert "mid[(4 * r + g) * 33 + 16 * t + c] = acc[t][r] * T3[0 + en * 32 + 16 * t + c];" in src
    assert "const double us = mid[c * 33 + 4 * step + g];" in src and "T0[" not in src
    # an intermediate that is not transient is stored as well as handed over
    src = operator_chain_source(TE, 32, 27, 1003, transient=False)
    assert src.count("__global__") == 1 and "mid[(4 * r + g) * 33 + 16 * t + c] = " in src
    assert "__builtin_nontemporal_store(acc[t][r] * T3[0 + en * 32 + 16 * t + c], a + 4 * r * 32 + 16 * t);" in src
    assert "applied to the first result on chip" in operator_chain_source(TE, 8, 8, 1002)


def test_pointwise_kernel_after_an_operator_kernel_is_folded_into_it(TE):
    E, nq, nd = 1005, 32, 27
    B, X, D = at.Tensor(nq, nd), at.Tensor(E, nd), at.Tensor(E, nq)
    U, V, Y = at.Tensor(E, nq), at.Tensor(E, nq), at.Tensor(E, nd)
    for transient in (True, False):
        U.SetTransient(transient)
        V.SetTransient(True)
        TE.BeginMultiKernelLaunch()
        TE("U_e_k = B_k_j X_e_j", U, B, X)
        TE("V_e_k = U_e_k D_e_k", V, U, D)
        TE("Y_e_i = B_k_i V_e_k", Y, B, V)
        src = TE.EndMultiKernelLaunchGetImplementation()
        # a stored U must reach device memory: nothing is folded then, and the group is an ordinary chain
        assert ("[0] U_e_k = B_k_j X_e_j ; V_e_k = U_e_k D_e_k" in src) == transient
        assert ("applied to the first result on chip" in src) == transient


def test_every_kind_of_generated_kernel_compiles_for_gfx950(TE, monkeypatch):
    import ctypes
    from acrotensor_amd import _capi
    lib = _capi.load()
    sources = list(generated_sources(TE))
    monkeypatch.setenv("ACRO_HIP_ONE_PASS", "1")
    sources.append(("split contraction, one launch",
                    TE.GetImplementation("S_i_j = A_n_i_j B_n", at.Tensor(3, 3), at.Tensor(70001, 3, 3), at.Tensor(70001))))
    monkeypatch.setenv("ACRO_HIP_OPERATOR_MFMA", "-1")
    sources.append(("operator schedule through scalar loads",
                    TE.GetImplementation("A_e_i1_i2 -= X_e_j1_j2 B_i1_i2_j1_j2", at.Tensor(79, 5, 6), at.Tensor(79, 4, 7), at.Tensor(5, 6, 4, 7))))
    for name, src in sources:
        assert "__global__" in src, name
        size = ctypes.c_size_t(0)
        rc = lib.acro_hip_compile(("unit_" + name.split(",")[0].replace(" ", "_")).encode(), src.encode(), ctypes.byref(size))
        assert rc == 0 and size.value > 0, (name, lib.acro_last_error().decode()[-2000:])


def test_bad_kernel_strings_fail_before_code_generation():
    TE = at.TensorEngine("HIP")
    with pytest.raises(at.AcroError):
        TE.GetImplementation("A_i = b_i", at.Tensor(3), at.Tensor(3))


def test_products_of_element_matrices_run_on_the_matrix_cores(TE, monkeypatch):
    """The product schedule (codegen_product.cpp): which products take it, how each factor reaches the instruction's
    operand layout, and what does not qualify."""
    def product(kernel, M, N, K, E=4096):
        ext = {"e": E, "i": M, "j": N, "k": K}
        lhs, rhs = kernel.replace("+=", "=").replace("-=", "=").split("=")
        tensors = [at.Tensor(*[ext[x] for x in tok.split("_")[1:]]) for tok in [lhs.split()[0]] + rhs.split()]
        return at.TensorEngine("HIP").GetImplementation(kernel, *tensors)

    # rows of a multiple of 128 bytes along the contracted index: the row factor straight into registers in pairs
    # (terms permuted), the column factor through LDS; four strips, one entry per workgroup of 256 lanes
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 64, 64, 64)
    assert "product schedule on the FP64 matrix cores: 64 x 64 by 64 x 64 per entry" in src
    assert "read straight into registers" in src and "(terms in pairs)" in src and "1 entry per workgroup of 256 lanes, LDS 32768 bytes" in src
    assert "const int k = 8 * u + 2 * g;" in src and src.count("__syncthreads()") == 3
    assert "acc[J] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[s], frag[(J * 16 + s) * 64 + g * 16 + acro_place(16 * J + c, k)], acc[J], 0, 0, 0);" in src
    assert "__builtin_nontemporal_store(v, d);" in src
    # other rows along the contracted index: every wavefront passes its strip, a contiguous range, through LDS
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 53, 53, 53)
    assert "strips through LDS" in src and "14 steps of four terms," in src and "LDS 28672 bytes" in src
    assert "const int x = j / 53, k = j % 53;" in src and '__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");' in src
    assert src.count("__syncthreads()") == 4
    # terms past the end are zero in both factors' fragments (53 = 13 * 4 + 1: three places of the last step)
    assert "fr[(13) * 64 + (1 + w) * 16 + (z & 15)] = 0.0;" in src and "fr[(blk * 14 + 13) * 64 + (1 + w) * 16 + (z & 15)] = 0.0;" in src
    # the row factor with the contracted index first: 128 contiguous bytes per term, straight into registers
    src = product("A_e_i_j = B_e_k_i C_e_k_j", 40, 40, 40)
    assert "row factor with the contracted index first, read straight into registers" in src and "a[s] = k < 40 ? rm[k * 40 + m] : 0.0;" in src
    # the column factor either way round, the factors in either order, accumulation into the result
    src = product("A_e_i_j -= C_e_j_k B_e_i_k", 37, 45, 20)
    assert "37 x 20 by 20 x 45 per entry" in src and "column factor with the contracted index last" in src
    assert "*d = *d - v;" in src and "nontemporal" not in src
    # small matrices: two entries per workgroup
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 31, 31, 31)
    assert "2 strips of 16 rows x 2 blocks of 16 columns" in src and "2 entries per workgroup of 256 lanes" in src
    # an odd number of doubles in the whole tensor: its last one is read on its own
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 17, 17, 17, E=4097)
    assert "if (at == 1184032L) cv[it].x = T2[1184032L];" in src
    # an element matrix applied to an element vector, rows that are no whole number of 32-byte pieces: a single column
    src = TE.GetImplementation("A_e_i = B_e_i_j C_e_j", at.Tensor(4096, 27), at.Tensor(4096, 27, 27), at.Tensor(4096, 27))
    assert "product schedule on the FP64 matrix cores: 27 x 27 by 27 x 1 per entry" in src and "2 strips of 16 rows x 1 blocks of 16 columns" in src
    for rows, cols in ((27, 32), (21, 21), (9, 45)):     # rows of whole pieces, short rows, few rows: the vector-ALU schedules
        assert "product schedule" not in TE.GetImplementation("A_e_i = B_e_i_j C_e_j", at.Tensor(4096, rows), at.Tensor(4096, rows, cols), at.Tensor(4096, cols))
    assert "product schedule" not in TE.GetImplementation("A_e_i = B_e_i_j C_j", at.Tensor(4096, 27), at.Tensor(4096, 27, 27), at.Tensor(27))
    # not this schedule: small matrices whose extents the staged schedule can split into blocks, 16 x 16 and smaller,
    # a shared factor, more than two factors, too few entries for e to be the batch index
    assert "product schedule" not in product("A_e_i_j = B_e_i_k C_e_k_j", 24, 24, 24)
    assert "product schedule" not in product("A_e_i_j = B_e_i_k C_e_k_j", 33, 33, 33)
    # (extents up to 32 that only three divides would get blocks of 3 x 3 there: those are taken, and so are whole blocks of 16)
    assert "product schedule on the FP64 matrix cores: 32 x 32 by 32 x 32" in product("A_e_i_j = B_e_i_k C_e_j_k", 32, 32, 32)
    assert "product schedule on the FP64 matrix cores: 27 x 27 by 27 x 27" in product("A_e_i_j = B_e_i_k C_e_k_j", 27, 27, 27)
    assert "product schedule on the FP64 matrix cores: 21 x 27 by 27 x 30" in product("A_e_i_j = B_e_i_k C_e_k_j", 21, 30, 27)
    assert "product schedule" not in product("A_e_i_j = B_e_i_k C_e_k_j", 16, 16, 16)
    assert "product schedule" not in TE.GetImplementation("A_e_i_j = B_e_i_k C_k_j", at.Tensor(4096, 40, 40), at.Tensor(4096, 40, 40), at.Tensor(40, 40))
    assert "product schedule" not in TE.GetImplementation("A_e_i_j = B_e_i_k C_e_k_j D_e", at.Tensor(4096, 40, 40), at.Tensor(4096, 40, 40),
                                                          at.Tensor(4096, 40, 40), at.Tensor(4096))
    assert "product schedule" not in product("A_e_i_j = B_e_i_k C_e_k_j", 50, 50, 50, E=30)
    # ... and it is a matrix-core schedule: off where those are refused
    monkeypatch.setenv("ACRO_HIP_TEST_PRIVATE_BYTES", "8,8")
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 64, 64, 64)
    assert "product schedule" not in src and "was refused" in src


def test_products_of_large_matrices_run_in_tiles_on_the_matrix_cores(TE, monkeypatch):
    """The tiled product schedule (codegen_product.cpp): products beyond one workgroup's reach and products without a
    batch index; how the result is split into tiles and what each form of the factors turns into."""
    def product(kernel, M, N, K, E=2048):
        ext = {"e": E, "i": M, "j": N, "k": K}
        lhs, rhs = kernel.replace("+=", "=").replace("-=", "=").split("=")
        tensors = [at.Tensor(*[ext[x] for x in tok.split("_")[1:]]) for tok in [lhs.split()[0]] + rhs.split()]
        return at.TensorEngine("HIP").GetImplementation(kernel, *tensors)

    # 128 x 128 per entry: four strips by four blocks per workgroup, four tiles per entry, chunks of 16 terms
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 128, 128, 128)
    assert "tiled product schedule on the FP64 matrix cores: 128 x 128 by 128 x 128 per entry, 2048 entries" in src
    assert "tiles of 64 rows x 64 columns (2 x 2 per entry), chunks of 16 terms through 16384 bytes of LDS, 8192 workgroups of 256 lanes" in src
    assert "__shared__ double fragA[1024];" in src and "__shared__ double fragB[1024];" in src
    # the lanes run along each factor's fastest dimension; values land in the instruction's operand order
    assert "const int kk = v % 16, rr = v / 16;" in src and "const int cc = v % 64, kk = v / 64;" in src
    assert "((rr / 16) * 4 + kk / 4) * 64 + (kk % 4) * 16 + ((rr + kk) & 15)" in src
    # nothing in the loop depends on the lane but a 32-bit offset: loads from a base that moves with the chunk, values
    # straight to LDS, the next chunk requested before the products; 16 divides the range, so no code for what is left
    assert "const int kBegin = 0, kEnd = 128;" in src and "unsigned aFrom[4], bFrom[4];" in src
    assert "const double *rk = Rm + k0, *ck = Cm + (long)k0 * 128;" in src and "ra[u] = rk[aFrom[u]];" in src and "fragA[aTo[u]] = ra[u];" in src
    assert src.index("const int k0 = kc + 16 < kWhole ? kc + 16 : kEnd - 16;") < src.index("__builtin_amdgcn_mfma_f64_16x16x4f64")
    assert src.count("__syncthreads()") == 2 and "__builtin_nontemporal_store(acc[J][q], d);" in src and "done" not in src
    assert "if (m >= 128" not in src                       # tiles without padding store without guards
    # extents that 16 does not divide, the factors stored the other way round, accumulation
    src = product("A_e_i_j += B_e_k_i C_e_j_k", 100, 70, 150)
    assert "100 x 150 by 150 x 70 per entry" in src and "row factor with the contracted index first, column factor with the contracted index last" in src
    assert "tiles of 64 rows x 80 columns (2 x 1 per entry)" in src and "workgroups of 256 lanes" in src
    assert "const int rr = v % 64, kk = v / 64;" in src and "const int kk = v % 16, cc = v / 16;" in src
    # rows and columns past the end read the last one (their results are not stored); the 6 terms after the whole chunks
    # are read as the last 16, and the 10 of them that the loop has added become zero on their way to LDS
    assert "const int row = r0 + rr < 100 ? r0 + rr : 99;" in src and "const int col = c0 + cc < 70 ? c0 + cc : 69;" in src
    assert "const int done = kWhole - (kEnd - 16);" in src and "fragA[aTo[u]] = v / 64 >= done ? ra[u] : 0.0;" in src
    assert "fragB[bTo[u]] = v % 16 >= done ? rb[u] : 0.0;" in src and src.count("__syncthreads()") == 3
    assert "if (m >= 100 || n >= 70) continue;" in src and "*d += acc[J][q];" in src and "nontemporal" not in src
    # no batch index: a plain matrix product; few tiles take half the height to fill the device
    src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(2048, 2048), at.Tensor(2048, 2048), at.Tensor(2048, 2048))
    assert "2048 x 2048 by 2048 x 2048, no batch index" in src and "tiles of 128 rows x 64 columns (16 x 32 per entry)" in src and "512 workgroups" in src
    src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(1024, 1024), at.Tensor(1024, 1024), at.Tensor(1024, 1024))
    assert "tiles of 64 rows x 64 columns (16 x 16 per entry)" in src and "768 workgroups of 256 lanes, the contracted range in 3 shares of 352 terms" in src
    # (a workgroup takes its chunks one after the other: with few tiles the contracted range is shared out as well, as far
    # as the partial sums and the second launch are worth it)
    src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(512, 512), at.Tensor(512, 512), at.Tensor(512, 512))
    assert "256 workgroups of 256 lanes, the contracted range in 4 shares of 128 terms" in src
    src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(512, 512), at.Tensor(512, 64), at.Tensor(64, 512))
    assert "64 workgroups of 256 lanes" in src and "shares" not in src
    src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(1536, 1536), at.Tensor(1536, 1536), at.Tensor(1536, 1536))
    assert "576 workgroups of 256 lanes" in src and "shares" not in src
    # few tiles, many terms (normal equations with more columns than the Gram schedule takes): the contracted range is
    # shared out as well, partial tiles go to the scratch buffer and a second kernel adds them in a fixed order
    src = TE.GetImplementation("A_i_j += B_n_i C_n_j", at.Tensor(128, 128), at.Tensor(262144, 128), at.Tensor(262144, 128))
    assert "tiles of 64 rows x 64 columns (2 x 2 per entry)" in src and "764 workgroups of 256 lanes, the contracted range in 191 shares of 1376 terms" in src
    assert "_partial(" in src and "double *__restrict__ scratch)" in src and "const int split = blockIdx.x / 4;" in src
    assert "scratch[((long)split * 1 + e) * 16384L + (long)m * 128 + n] = acc[J][q];" in src
    # (the second kernel: four lanes per output where the outputs alone are too few to keep the loads in flight)
    assert "for (int w = part; w < 191; w += 4) t += scratch[w * 16384L + o];" in src and "result[0L + o] = result[0L + o] + t;" in src
    src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(512, 512), at.Tensor(512, 512), at.Tensor(512, 512))
    assert "for (int w = 0; w < 4; ++w) t += scratch[w * 262144L + o];" in src
    # fewer than 64 x 64 outputs, also fewer than 16 rows or columns, where the contracted range is long (1 024 terms and
    # more) and there are 64 outputs or more: the generic schedule would give the whole range to single lanes
    for rows, cols, terms in ((32, 32, 100000), (8, 100, 100000), (100, 8, 100000), (15, 15, 100000), (8, 31, 100000), (3, 300, 5000)):
        src = TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(rows, cols), at.Tensor(rows, terms), at.Tensor(terms, cols))
        assert "tiled product schedule" in src and "shares of" in src, (rows, cols, terms)
    assert "tiled" not in TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(32, 32), at.Tensor(32, 1000), at.Tensor(1000, 32))
    assert "reduction schedule" in TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(4, 4), at.Tensor(4, 100000), at.Tensor(100000, 4))
    # 65 to 128 rows or columns per entry, and small matrices with more than 128 terms
    assert "tiled product schedule" in product("A_e_i_j = B_e_i_k C_e_k_j", 72, 72, 72)
    assert "tiled product schedule" in product("A_e_i_j = B_e_i_k C_e_k_j", 32, 48, 200)
    # entries fewer than rows: the entry index is still the first one
    assert "tiled product schedule" in product("A_e_i_j = B_e_i_k C_e_k_j", 128, 128, 128, E=10)
    # not this schedule: what the product schedule takes, tiny matrices, a shared factor
    assert "tiled" not in product("A_e_i_j = B_e_i_k C_e_k_j", 64, 64, 64)
    assert "tiled" not in product("A_e_i_j = B_e_i_k C_e_k_j", 8, 100, 100)
    assert "tiled" not in TE.GetImplementation("A_e_i_j = B_e_i_k C_k_j", at.Tensor(64, 100, 100), at.Tensor(64, 100, 100), at.Tensor(100, 100))
    assert "tiled" not in TE.GetImplementation("A_i_j = B_i_k C_k_j", at.Tensor(32, 32), at.Tensor(32, 32), at.Tensor(32, 32))
    # ... and it is a matrix-core schedule: off where those are refused
    monkeypatch.setenv("ACRO_HIP_TEST_PRIVATE_BYTES", "8,8")
    src = product("A_e_i_j = B_e_i_k C_e_k_j", 128, 128, 128)
    assert "tiled product schedule" not in src and "was refused" in src


def test_operands_read_once_in_whole_lines_take_the_non_temporal_hint(TE, monkeypatch):
    # the mass apply's element vector: 64 values per entry, the lanes on its two fastest dimensions; the geometric factors,
    # five doubles per lane at a stride, keep ordinary loads
    src = chain_source(TE, workloads.config4(E=64), transient=True)
    assert "__builtin_nontemporal_load(&T2[o_k0v1 + 0])" in src and "__builtin_nontemporal_load(&T6[" not in src
    assert "= T6[o_k3v0 + 0];" in src
    # the diffusion apply's element vector is read by two kernels of the group: ordinary loads
    src = chain_source(TE, workloads.config5(E=8), transient=True)
    assert "__builtin_nontemporal_load" not in src
    # kernels without contraction whose operands lie in memory as the result does
    src = TE.GetImplementation("A_e_i = B_e_i C_e_i", at.Tensor(4096, 16), at.Tensor(4096, 16), at.Tensor(4096, 16))
    assert src.count("__builtin_nontemporal_load(&T") == 2
    # ... not an operand whose values go to several work items, not the batch index last
    assert "__builtin_nontemporal_load" not in TE.GetImplementation("A_e_i_j = B_e_i C_e_j", at.Tensor(4096, 8, 8), at.Tensor(4096, 8), at.Tensor(4096, 8))
    assert "__builtin_nontemporal_load" not in TE.GetImplementation("A_i_e = B_i_e C_i_e", at.Tensor(16, 4096), at.Tensor(16, 4096), at.Tensor(16, 4096))
    # a contraction shared by lanes along rows of whole lines; rows of 100 doubles share lines
    assert "__builtin_nontemporal_load" in TE.GetImplementation("A_e = B_e_n", at.Tensor(4096), at.Tensor(4096, 1024))
    assert "__builtin_nontemporal_load" not in TE.GetImplementation("A_e = B_e_n", at.Tensor(4096), at.Tensor(4096, 100))
    # reductions: the streaming forms, not the pencil form
    assert "__builtin_nontemporal_load" in TE.GetImplementation("S_i = A_n_i", at.Tensor(64), at.Tensor(1 << 16, 64))
    assert "__builtin_nontemporal_load" not in TE.GetImplementation("S_i_j = A_n_i_j B_n", at.Tensor(3, 3), at.Tensor(1 << 16, 3, 3), at.Tensor(1 << 16))
    # Gram sums with rows of whole lines, factors of element-matrix products that are whole lines per entry
    assert "__builtin_nontemporal_load(&b[16 * ti])" in TE.GetImplementation("A_i_j = B_e_i C_e_j", at.Tensor(32, 32), at.Tensor(1 << 16, 32), at.Tensor(1 << 16, 32))
    assert "__builtin_nontemporal_load" not in TE.GetImplementation("A_i_j = B_e_i C_e_j", at.Tensor(24, 24), at.Tensor(1 << 16, 24), at.Tensor(1 << 16, 24))
    assert "__builtin_nontemporal_load" in TE.GetImplementation("A_e_i_j = B_e_i_k C_e_k_j", at.Tensor(512, 32, 32), at.Tensor(512, 32, 32), at.Tensor(512, 32, 32))
    assert "__builtin_nontemporal_load" not in TE.GetImplementation("A_e_i_j = B_e_i_k C_e_k_j", at.Tensor(512, 33, 33), at.Tensor(512, 33, 33), at.Tensor(512, 33, 33))
    monkeypatch.setenv("ACRO_HIP_NT_LOADS", "-1")
    assert "__builtin_nontemporal_load" not in chain_source(at.TensorEngine("HIP"), workloads.config4(E=64), transient=True)


def test_long_contractions_that_no_schedule_takes_are_shared_out_over_workgroups(TE, monkeypatch):
    # more than 128 outputs whose big operand does not stream once, few long rows, interleaved layouts: the generic plan
    # would leave hundreds of terms to each of few lanes
    src = TE.GetImplementation("A_i_j += B_i_e C_j", at.Tensor(12, 16), at.Tensor(12, 1 << 20), at.Tensor(16))
    assert "reduction schedule: 192 output entries" in src and "four outputs per workgroup" in src
    src = TE.GetImplementation("A_e += B_i C_e_i", at.Tensor(2048), at.Tensor(8192), at.Tensor(2048, 8192))
    assert "reduction schedule: 2048 output entries" in src and "const int o = blockIdx.x * 256 + threadIdx.x;" in src
    # outputs and terms numbered in the big operand's memory order: D_k_j_e_i has i fastest, then e
    src = TE.GetImplementation("A_i_k = B_j_k_l C_e D_k_j_e_i", at.Tensor(5, 9), at.Tensor(16, 9, 20), at.Tensor(4096), at.Tensor(9, 16, 4096, 5))
    assert "const int i_k = (int)(o / 5);" in src and "const int i_i = (int)((o / 1) % 5);" in src
    assert "const int i_e = (int)((c / 1) % 4096);" in src
    # many lanes in the generic plan: it keeps the kernel
    assert "reduction schedule" not in TE.GetImplementation("A_j_k += B_j_k_i C_j_i_e", at.Tensor(7, 8192), at.Tensor(7, 8192, 512), at.Tensor(7, 512, 100))
    monkeypatch.setenv("ACRO_HIP_RED_FALLBACK", "-1")
    assert "reduction schedule" not in at.TensorEngine("HIP").GetImplementation("A_i_j += B_i_e C_j", at.Tensor(12, 16), at.Tensor(12, 1 << 20), at.Tensor(16))


def test_operands_that_carry_a_contraction_index_alone_are_summed_first(TE):
    src = TE.GetImplementation("A_e = B_e_j C_e_i", at.Tensor(4096), at.Tensor(4096, 32), at.Tensor(4096, 27))
    assert "_F1_e = B_e_j" in src and "_F2_e = C_e_i" in src and "A_e = _F1_e _F2_e   (steps of: A_e = B_e_j C_e_i)" in src
    src = TE.GetImplementation("A_e_l = B_i_l C_e_j_k", at.Tensor(4096, 10), at.Tensor(20, 10), at.Tensor(4096, 64, 9))
    assert "_F1_e = C_e_j_k" in src and "A_e_l = B_i_l _F1_e" in src
    # nothing to sum first: both operands carry the contraction index; too little work: as written
    assert "steps of" not in TE.GetImplementation("A_e_i = B_e_i_j C_e_j", at.Tensor(4096, 8), at.Tensor(4096, 8, 8), at.Tensor(4096, 8))
    assert "steps of" not in TE.GetImplementation("A_e = B_e_j C_e_i", at.Tensor(4096), at.Tensor(4096, 4), at.Tensor(4096, 4))
    # short sums per entry: products into an LDS tile with the lanes along memory, then a lane per sum
    src = TE.GetImplementation("A_e = B_e_i C_e_i", at.Tensor(4096), at.Tensor(4096, 27), at.Tensor(4096, 27))
    assert "_F1_e_i = B_e_i C_e_i" in src and "A_e = _F1_e_i   (steps of:" in src
    assert "steps of" in TE.GetImplementation("A_e = B_e_i", at.Tensor(4096), at.Tensor(4096, 9))
    for row in (3, 5, 16, 100):
        assert "steps of" not in TE.GetImplementation("A_e = B_e_i", at.Tensor(4096), at.Tensor(4096, row))
    # a vector applied from the left to an element matrix of few columns: the second step adds down the columns of the tile
    src = TE.GetImplementation("A_e_j = B_e_i_j C_e_i", at.Tensor(4096, 2), at.Tensor(4096, 27, 2), at.Tensor(4096, 27))
    assert "_F1_e_i_j = B_e_i_j C_e_i" in src and "A_e_j = _F1_e_i_j   (steps of:" in src
    assert "steps of" not in TE.GetImplementation("A_e_j = B_e_i_j C_i", at.Tensor(4096, 2), at.Tensor(4096, 64, 2), at.Tensor(64))
    assert "steps of" not in TE.GetImplementation("A_e_j = B_e_i_j C_e_i", at.Tensor(4096, 8), at.Tensor(4096, 27, 8), at.Tensor(4096, 27))
    # a contraction shared by lanes is numbered as the terms lie in the streaming operand
    src = TE.GetImplementation("A_e = B_i_j C_e_j_i", at.Tensor(4096), at.Tensor(20, 8), at.Tensor(4096, 8, 20))
    assert "contraction shared by" in src and "lanes()=16" in src
