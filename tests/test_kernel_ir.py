"""Kernel-string parser and dimensioned-kernel bookkeeping, through the C ABI's host-only introspection call.

Expectations are the literal ones of the reference's unittest/kernel/test_TensorKernel.cpp:15-160 and
unittest/kernel/test_DimensionedKernel.cpp:17-77, plus the reference's own answers (oracle/_ref) where built."""
import pytest

import acrotensor_amd as at

STIFF3D = "S_e_i1_i2_i3_j1_j2_j3 =B_i1_j1_k1_m_nB_i2_j2_k2_m_nB_i3_j3_k3_m_n D_e_k1_k2_k3_m_n"
STIFF3D_SHAPES = [(10, 5, 5, 5, 5, 5, 5), (5, 5, 5, 3, 3), (5, 5, 5, 3, 3), (5, 5, 5, 3, 3), (10, 5, 5, 5, 3, 3)]


def describe(kernel, shapes):
    return at.describe_kernels([kernel], [shapes])


@pytest.mark.parametrize("bad", ["Blah", "Blah=", "Blah=Alah", "BLA1h=Alah", "B_lah=A_lah_", "B_lah_=A_lah",
                                 "a_lah_=A_lah", "", "A_i", "A_i=", "A_i==B_i", "A_i+B_i", "A_i=B_I", "A_i=b_i",
                                 "A_i=B_i-", "A__i=B_i"])
def test_unparsable_strings_are_rejected(bad):
    with pytest.raises(at.AcroError):
        describe(bad, [(3,), (3,)])


def test_parsable_string():
    d = describe("B_lah=A_lah", [(3,), (3,)])
    assert d["kernels"][0]["name"] == "B_laheqA_lah"


@pytest.mark.parametrize("kernel,name", [("BA_i=A_j", "BA_ieqA_j"), ("B1_i=CB_jBr_j", "B1_ieqCB_jBr_j"),
                                         ("A_i += B_i", "A_ipeB_i"), ("A_i -= B_i C_i", "A_imeB_iC_i")])
def test_name_string(kernel, name):
    nin = name.count("_") - 1
    d = describe(kernel, [(3,)] * (1 + nin))
    assert d["kernels"][0]["name"] == name


def test_elementwise_product():
    k = describe("A_i=B_iC_i", [(3,), (3,), (3,)])["kernels"][0]
    assert k["all_indices"] == ["i"] and k["contraction_indices"] == []
    assert [v["loop_nums"] for v in k["vars"]] == [[0], [0], [0]]
    assert (k["flat_size"], k["out_size"], k["cont_size"]) == (3, 3, 1)
    assert k["out_storage_inner"][1] == 3 and k["in_storage_inner"][1] == 6


def test_contraction_with_transposed_operands():
    k = describe("A_i=B_s_iC_i_s", [(3,), (3, 3), (3, 3)])["kernels"][0]
    assert k["all_indices"] == ["i", "s"] and k["contraction_indices"] == ["s"]
    assert [v["loop_nums"] for v in k["vars"]] == [[0], [1, 0], [0, 1]]
    assert (k["flat_size"], k["out_size"], k["cont_size"]) == (9, 3, 3)
    assert k["out_storage_inner"][1:3] == [1, 3] and k["in_storage_inner"][1:3] == [6, 18]


def test_contraction_with_invariant_operand():
    k = describe("A_i=B_s_iC_i", [(3,), (3, 3), (3,)])["kernels"][0]
    assert (k["flat_size"], k["out_size"], k["cont_size"]) == (9, 3, 3)
    assert k["out_storage_inner"][1:3] == [1, 3] and k["in_storage_inner"][1:3] == [4, 12]


def test_multi_character_indices():
    k = describe("A_i1_i2=B_i1_i2_sum1", [(2, 3), (2, 3, 4)])["kernels"][0]
    assert k["all_indices"] == ["i1", "i2", "sum1"] and k["contraction_indices"] == ["sum1"]


def test_3d_stiffness_kernel():
    k = describe(STIFF3D, STIFF3D_SHAPES)["kernels"][0]
    assert k["all_indices"] == ["e", "i1", "i2", "i3", "j1", "j2", "j3", "k1", "m", "n", "k2", "k3"]
    assert k["contraction_indices"] == ["k1", "m", "n", "k2", "k3"]
    assert len(k["vars"]) == 5
    assert (k["flat_size"], k["out_size"], k["cont_size"]) == (175781250, 156250, 1125)


def test_white_space_is_ignored():
    a = describe("A_i = B_i_j  C_j", [(3,), (3, 4), (4,)])["kernels"][0]
    b = describe("A_i=B_i_jC_j", [(3,), (3, 4), (4,)])["kernels"][0]
    assert a["name"] == b["name"] and a["dimensioned_name"] == b["dimensioned_name"]


def test_incompatible_extents_are_rejected():
    with pytest.raises(at.AcroError, match="Incompatible tensor dimensions"):
        describe("A_i=B_iC_i", [(3,), (3,), (2,)])
    with pytest.raises(at.AcroError, match="rank"):
        describe("A_i=B_i_j", [(3,), (3,)])


def test_dimensioned_names_match_the_documented_form():
    d = describe("T1_e_q_j_k = B_q_i X_e_i_j_k", [(4096, 5, 4, 4), (5, 4), (4096, 4, 4, 4)])["kernels"][0]
    assert d["dimensioned_name2"] == "T1_e_q_j_keqB_q_iX_e_i_j_k__dim_4096_5_4_4_4"
    assert d["dimensioned_name"] == "T1_e_q_j_keqB_q_iX_e_i_j_k__4096_5_4_4_4"


def mass_chain(E):
    kernels = ["T1_e_q_j_k = B_q_i X_e_i_j_k", "T2_e_q_r_k = B_r_j T1_e_q_j_k", "T3_e_q_r_s = B_s_k T2_e_q_r_k",
               "U_e_q_r_s = D_e_q_r_s T3_e_q_r_s", "V1_e_i_r_s = B_q_i U_e_q_r_s", "V2_e_i_j_s = B_r_j V1_e_i_r_s",
               "Y_e_i_j_k = B_s_k V2_e_i_j_s"]
    B, X, D = (5, 4), (E, 4, 4, 4), (E, 5, 5, 5)
    T1, T2, T3, V1, V2 = (E, 5, 4, 4), (E, 5, 5, 4), (E, 5, 5, 5), (E, 4, 5, 5), (E, 4, 4, 5)
    shapes = [[T1, B, X], [T2, B, T1], [T3, B, T2], [D, D, T3], [V1, B, D], [V2, B, V1], [X, B, V2]]
    return kernels, shapes


def test_multi_kernel_of_the_mass_apply_chain():
    kernels, shapes = mass_chain(64)
    m = at.describe_kernels(kernels, shapes)["multi"]
    assert m["shared_outer"] == ["e"]
    assert m["loop_indices"] == ["e", "q", "j", "k", "i", "r", "s"]
    assert m["unique_vars"] == ["T1", "B", "X", "T2", "T3", "U", "D", "V1", "V2", "Y"]
    assert m["loop_dims"] == [64, 5, 4, 4, 4, 5, 5]


def test_shared_outer_indices_are_ordered_by_extent_then_name():
    m = at.describe_kernels(["A_b_a_c = B_a_b_c_k C_k"], [[(7, 9, 7), (9, 7, 7, 2), (2,)]])["multi"]
    assert m["shared_outer"] == ["a", "b", "c"]          # a is largest; b and c tie and sort by name
    assert m["loop_indices"] == ["a", "b", "c", "k"]


CASES = [
    ("A_i=B_iC_i", [(3,), (3,), (3,)]),
    ("A_i=B_s_iC_i_s", [(3,), (3, 3), (3, 3)]),
    ("S_i_j = A_n_i_j B_n", [(3, 3), (100, 3, 3), (100,)]),
    ("A_b_a_c = B_a_b_c_k C_k", [(7, 9, 7), (9, 7, 7, 2), (2,)]),
    ("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s",
     [(8, 3, 3, 3, 3, 3, 3)] + [(4, 3)] * 6 + [(8, 4, 4, 4)]),
    (STIFF3D, STIFF3D_SHAPES),
]


@pytest.mark.parametrize("kernel,shapes", CASES)
def test_against_the_compiled_reference(reference, kernel, shapes):
    ref = reference.describe(kernel, shapes)
    d = at.describe_kernels([kernel], [shapes])
    k, m = d["kernels"][0], d["multi"]
    assert ",".join(k["all_indices"]) == ref["all"]
    assert ",".join(k["contraction_indices"]) == ref["contr"]
    assert ",".join(m["loop_indices"]) == ref["loops"]
    assert ",".join(str(x) for x in m["loop_dims"]) == ref["dims"]
    assert k["dimensioned_name"] == ref["dname"] and k["dimensioned_name2"] == ref["dname2"]
    assert (str(k["flat_size"]), str(k["out_size"]), str(k["cont_size"])) == (ref["flat"], ref["out"], ref["cont"])
    assert reference.name_string(kernel) == k["name"]
