// Exercises the C++ API (the reference's own boundary) exactly as a user of the reference would write it:
// acro::Tensor / SliceTensor / IndexMapping / TensorEngine with the "HIP" policy.  Sections follow the
// reference's unittest/kernel/test_TensorEngine.cpp and unittest/tensor/test_Tensor.cpp; expectations are the
// closed forms those tests use.  "host" runs what needs no device, "gpu" runs everything.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>

#include "AcroTensor.hpp"

using namespace acro;

static int g_failures = 0;
static int g_checks = 0;

#define CHECK(cond)                                                        \
    do                                                                     \
    {                                                                      \
        ++g_checks;                                                        \
        if (!(cond))                                                       \
        {                                                                  \
            ++g_failures;                                                  \
            std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond);  \
        }                                                                  \
    } while (0)

static bool throwsError(const std::function<void()> &f)
{
    try
    {
        f();
    }
    catch (const std::runtime_error &)
    {
        return true;
    }
    return false;
}

#define CHECK_THROWS(stmt) CHECK(throwsError([&] { stmt; }))
#define CHECK_NOTHROW(stmt) CHECK(!throwsError([&] { stmt; }))

static bool approx(double a, double b)
{
    return std::fabs(a - b) <= 1e-12 * (1.0 + std::fabs(b));
}

static void hostTests()
{
    std::printf("host: tensors\n");
    CHECK_THROWS(Tensor(0));
    CHECK_THROWS(Tensor(3, -1));
    Tensor T(2, 3, 4);
    CHECK(T.GetRank() == 3 && T.GetSize() == 24 && T.GetDim(1) == 3 && T.GetStride(0) == 12);
    for (size_t i = 0; i < T.GetSize(); ++i) T[i] = i;
    CHECK(T(1, 2, 3) == 23.0 && T.GetRawIndex(1, 0, 2) == 14);
    T.Reshape(4, 6);
    CHECK(T.GetRank() == 2 && T(3, 5) == 23.0);
    CHECK_THROWS(T.Reshape(5, 5));
    CHECK_THROWS(T.Init(3));  // second initialisation
    Tensor late;
    CHECK(!late.IsInitialized());
    late.Init(2, 2);
    CHECK(late.IsInitialized() && late.GetSize() == 4);

    double buffer[6] = {0, 1, 2, 3, 4, 5};
    Tensor ext(2, 3, buffer);
    ext.Mult(2.0);
    CHECK(buffer[5] == 10.0);
    CHECK_THROWS(Tensor(2, 3, nullptr, buffer));        // device-only tensors are not supported
    CHECK_THROWS(Tensor(2, 3, buffer, nullptr, true));  // cannot be "on GPU" without a device pointer

    std::printf("host: slices\n");
    Tensor P(3, 4, 5);
    for (size_t i = 0; i < P.GetSize(); ++i) P[i] = i;
    SliceTensor S(P, 2), S2(P, 1, 3);
    CHECK(S.GetRank() == 2 && S.GetDim(0) == 4 && S(1, 2) == P(2, 1, 2));
    CHECK(S2.GetRank() == 1 && S2(4) == P(1, 3, 4));
    S.Set(-1.0);
    CHECK(P(2, 3, 4) == -1.0 && P(1, 3, 4) == 39.0);
    CHECK_THROWS(SliceTensor(P, 0, 0, 0));
    CHECK_THROWS(S.Retarget(buffer));

    std::printf("host: kernels\n");
    CHECK_THROWS(TensorKernel("Blah=Alah"));
    CHECK_THROWS(TensorKernel("B_lah=A_lah_"));
    CHECK_THROWS(TensorKernel("a_lah_=A_lah"));
    TensorKernel K("A_i=B_s_iC_i_s");
    CHECK(K.AllIndexNames.size() == 2 && K.ContractionIndexNames.size() == 1 && K.ContractionIndexNames[0] == "s");
    CHECK(K.GetVarDimLoopNum(0, 0) == 1 && K.GetVarDimLoopNum(0, 1) == 0 && !K.IsVarDependentOnLoop(-1, 1));
    CHECK(K.GetNameString() == "A_ieqB_s_iC_i_s");
    Tensor o3(3), m33(3, 3);
    std::vector<Tensor *> ins = {&m33, &m33};
    DimensionedKernel DK(&K, &o3, ins);
    CHECK(DK.GetFlatIdxSize() == 9 && DK.GetOutIdxSize() == 3 && DK.GetContIdxSize() == 3);
    CHECK(DK.GetInputStorageReqForInnerLoops(2) == 18);

    std::printf("host: index mapping\n");
    IndexMapping M(4, 8);
    const int map[8] = {3, 1, 2, 3, 0, 1, 1, 2};
    for (int i = 0; i < 8; ++i) M[i] = map[i];
    CHECK_THROWS(M.GetInvMap());
    M.ComputeInverse();
    CHECK(M.GetInvMap()[0] == 4 && M.GetInvMap()[1] == 1 && M.GetInvMapOffsets()[4] == 8);

    std::printf("host: engine\n");
    CHECK_THROWS(TensorEngine("NoSuchPolicy"));
    CHECK_THROWS(TensorEngine("CPUInterpreted"));  // this library never computes on the host
    TensorEngine TE("HIP");
    CHECK(TE.GetExecType() == "HIP");
    Tensor A(16, 3), B(16, 3, 5), C(5);
    std::string src = TE.GetImplementation("A_e_i = B_e_i_j C_j", A, B, C);
    CHECK(src.find("__global__") != std::string::npos);
    CHECK_THROWS(TE.EndMultiKernelLaunch());
    Tensor noinit;
    CHECK_THROWS(TE.GetImplementation("A_e_i = B_e_i_j C_j", A, B, noinit));
}

static void gpuTests()
{
    TensorEngine TE("HIP");
    CHECK(TE.IsGPUAvailable());

    std::printf("gpu: residency\n");
    {
        Tensor T(10, 10);
        T.Set(3.0);
        T.MapToGPU();
        CHECK(T.IsMappedToGPU() && !T.IsOnGPU());
        CHECK_THROWS(T.MapToGPU());
        T.SwitchToGPU();
        T.Set(9.0);
        CHECK(T(0, 0) == 3.0);
        T.MoveFromGPU();
        CHECK(T(9, 9) == 9.0 && !T.IsOnGPU());
        T.UnmapFromGPU();
        CHECK(!T.IsMappedToGPU());
    }

    std::printf("gpu: README example\n");
    {
        const int n = 1000;
        Tensor A(n, 3, 3), B(n), S(3, 3);
        for (size_t i = 0; i < A.GetSize(); ++i) A[i] = i % 7;
        B.Set(1.0);
        A.MapToGPU();
        A.MoveToGPU();
        B.MoveToGPU();
        S.SwitchToGPU();
        TE("S_i_j = A_n_i_j B_n", S, A, B);
        S.MoveFromGPU();
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j)
            {
                double sum = 0.0;
                for (int k = 0; k < n; ++k) sum += A(k, i, j);
                CHECK(S(i, j) == sum);
            }
    }

    std::printf("gpu: basic computations\n");
    {
        Tensor out3(3), out33(3, 3), in3(3), in33(3, 3);
        for (int i = 0; i < 9; ++i) in33[i] = i;
        in3(0) = 1.0;
        in3(1) = 2.0;
        in3(2) = 3.0;
        CHECK_THROWS(TE("A_i=B_iC_i", out3, in3, out33));
        TE("A_i=B_i", out3, in3);
        out3.MoveFromGPU();
        CHECK(out3(0) == 1.0 && out3(2) == 3.0);
        TE("A_i=B_i_i", out3, in33);
        out3.MoveFromGPU();
        CHECK(out3(0) == 0.0 && out3(1) == 4.0 && out3(2) == 8.0);
        TE("A_i=B_j_j", out3, in33);
        out3.MoveFromGPU();
        CHECK(out3(0) == 12.0 && out3(2) == 12.0);
        TE("A_i = C_i_j B_j", out3, in33, in3);
        out3.MoveFromGPU();
        CHECK(out3(0) == 8.0 && out3(1) == 26.0 && out3(2) == 44.0);
        TE("A_i_j=B_j_i", out33, in33);
        out33.MoveFromGPU();
        CHECK(out33(0, 2) == 6.0 && out33(2, 1) == 5.0);
        TE("A_m_n=B_m_j B_n_j", out33, in33, in33);
        out33.MoveFromGPU();
        CHECK(out33(0, 0) == 5.0 && out33(1, 2) == 86.0);
    }

    std::printf("gpu: multi kernel launch\n");
    {
        Tensor A(3), B1(3), B2(3), C(3, 3);
        B1(0) = 1.0;
        B1(1) = 2.0;
        B1(2) = 3.0;
        B2.Set(1.0);
        C.Set(1.0);
        TE.BeginMultiKernelLaunch();
        TE("A_i = B1_i", A, B1);
        TE("A_i = C_i_j B2_j", A, C, B2);
        TE.EndMultiKernelLaunch();
        A.MoveFromGPU();
        CHECK(A(0) == 3.0 && A(1) == 3.0 && A(2) == 3.0);
    }

    std::printf("gpu: mass apply chain with transient intermediates\n");
    {
        const int E = 37;
        Tensor Bm(5, 4), X(E, 4, 4, 4), D(E, 5, 5, 5), Y(E, 4, 4, 4);
        Tensor T1(E, 5, 4, 4), T2(E, 5, 5, 4), T3(E, 5, 5, 5), U(E, 5, 5, 5), V1(E, 4, 5, 5), V2(E, 4, 4, 5);
        for (size_t i = 0; i < Bm.GetSize(); ++i) Bm[i] = std::sin(1.0 + i);
        for (size_t i = 0; i < X.GetSize(); ++i) X[i] = std::cos(0.1 * i);
        for (size_t i = 0; i < D.GetSize(); ++i) D[i] = 1.0 + 0.5 * std::sin(0.3 * i);
        for (Tensor *t : {&T1, &T2, &T3, &U, &V1, &V2}) t->SetTransient(true);
        TE.BeginMultiKernelLaunch();
        TE("T1_e_q_j_k = B_q_i X_e_i_j_k", T1, Bm, X);
        TE("T2_e_q_r_k = B_r_j T1_e_q_j_k", T2, Bm, T1);
        TE("T3_e_q_r_s = B_s_k T2_e_q_r_k", T3, Bm, T2);
        TE("U_e_q_r_s = D_e_q_r_s T3_e_q_r_s", U, D, T3);
        TE("V1_e_i_r_s = B_q_i U_e_q_r_s", V1, Bm, U);
        TE("V2_e_i_j_s = B_r_j V1_e_i_r_s", V2, Bm, V1);
        TE("Y_e_i_j_k = B_s_k V2_e_i_j_s", Y, Bm, V2);
        TE.EndMultiKernelLaunch();
        Y.MoveFromGPU();
        // dense definition for two elements
        double worst = 0.0, scale = 0.0;
        for (int e : {0, E - 1})
            for (int i = 0; i < 4; ++i)
                for (int j = 0; j < 4; ++j)
                    for (int k = 0; k < 4; ++k)
                    {
                        double sum = 0.0;
                        for (int q = 0; q < 5; ++q)
                            for (int r = 0; r < 5; ++r)
                                for (int s = 0; s < 5; ++s)
                                {
                                    double t = 0.0;
                                    for (int l = 0; l < 4; ++l)
                                        for (int m = 0; m < 4; ++m)
                                            for (int n = 0; n < 4; ++n) t += Bm(q, l) * Bm(r, m) * Bm(s, n) * X(e, l, m, n);
                                    sum += Bm(q, i) * Bm(r, j) * Bm(s, k) * D(e, q, r, s) * t;
                                }
                        worst = std::fmax(worst, std::fabs(sum - Y(e, i, j, k)));
                        scale = std::fmax(scale, std::fabs(sum));
                    }
        CHECK(worst <= 1e-12 * scale);
    }

    std::printf("gpu: inverse, determinant, scatter, gather\n");
    {
        const int n = 100;
        Tensor A(n, 3, 3), Ainv(n, 3, 3), Adet(n), I(n, 3, 3);
        for (int b = 0; b < n; ++b)
            for (int i = 0; i < 3; ++i)
                for (int j = 0; j < 3; ++j) A(b, i, j) = (i == j ? 2.0 : 0.0) + 0.1 * std::sin(b + 3 * i + j);
        TE.BatchMatrixInvDet(Ainv, Adet, A);
        TE("I_b_i_k = TI_b_j_i T_b_j_k", I, Ainv, A);  // the 3x3 "inverse" is laid out transposed
        I.MoveFromGPU();
        bool identity = true;
        for (int b = 0; b < n; ++b)
            for (int i = 0; i < 3; ++i)
                for (int j = 0; j < 3; ++j) identity = identity && approx(I(b, i, j) + 1.0, (i == j ? 2.0 : 1.0));
        CHECK(identity);
        // the same two steps recorded as one launch: the inverse becomes a kernel of the group and stays in registers
        Tensor Ainv2(n, 3, 3), Adet2(n), I2(n, 3, 3);
        Ainv2.SetTransient(true);
        TE.BeginMultiKernelLaunch();
        TE.BatchMatrixInvDet(Ainv2, Adet2, A);
        TE("I_b_i_k = TI_b_j_i T_b_j_k", I2, Ainv2, A);
        TE.EndMultiKernelLaunch();
        CHECK(TE.GetLastImplementation().find("(matrix inverse)") != std::string::npos);
        CHECK(TE.GetLastImplementation().find("TI<-registers") != std::string::npos);
        I2.MoveFromGPU();
        Adet2.MoveFromGPU();
        Adet.MoveFromGPU();
        bool same = true;
        for (int b = 0; b < n; ++b)
        {
            same = same && Adet2(b) == Adet(b);
            for (int i = 0; i < 3; ++i)
                for (int j = 0; j < 3; ++j) same = same && I2(b, i, j) == I(b, i, j);
        }
        CHECK(same);
        Tensor bad(n, 4, 4);
        CHECK_THROWS(TE.BatchMatrixInverse(bad, bad));

        IndexMapping M(6, 8);
        const int map[8] = {0, 1, 2, 3, 4, 5, 1, 3};
        for (int i = 0; i < 8; ++i) M[i] = map[i];
        Tensor small(6), big(8), back(6);
        for (int i = 0; i < 6; ++i) small(i) = 10.0 * i;
        TE.FlatIndexedScatter(big, small, M);
        big.MoveFromGPU();
        CHECK(big(6) == 10.0 && big(7) == 30.0);
        for (int i = 0; i < 8; ++i) big(i) = i + 1.0;
        TE.FlatIndexedSumGather(back, big, M);
        back.MoveFromGPU();
        CHECK(back(1) == 9.0 && back(3) == 12.0 && back(5) == 6.0);
        // a scatter recorded in a multi-kernel launch, result transient: the kernel reads `small` through the map
        Tensor gathered(8), squares(8);
        gathered.SetTransient(true);
        TE.BeginMultiKernelLaunch();
        TE.FlatIndexedScatter(gathered, small, M);
        TE("Q_i = G_i G_i", squares, gathered, gathered);
        TE.EndMultiKernelLaunch();
        CHECK(TE.GetLastImplementation().find("G<-gathered") != std::string::npos);
        squares.MoveFromGPU();
        CHECK(squares(0) == 0.0 && squares(5) == 2500.0 && squares(6) == 100.0 && squares(7) == 900.0);
    }

    std::printf("gpu: externally owned device memory\n");
    {
        Tensor owner(8);
        owner.MapToGPU();
        double host[8] = {0, 1, 2, 3, 4, 5, 6, 7}, result[8];
        {
            Tensor wrap(8, host, owner.GetDeviceData(), false);  // caller's buffers, device copy not current
            Tensor out(8, result);
            CHECK(wrap.IsMappedToGPU() && !wrap.IsOnGPU());
            TE("A_i = B_i", out, wrap);
            CHECK(wrap.IsOnGPU());
            out.MoveFromGPU();
            out.UnmapFromGPU();
        }
        CHECK(result[7] == 7.0 && owner.IsMappedToGPU());  // the wrapper did not free the caller's allocation
    }

    std::printf("gpu: recorded launch sequence, page-locked host buffers\n");
    {
        Tensor::SetPinnedHostAllocation(true);
        Tensor A(64, 3), B(64, 3), C(3);
        Tensor::SetPinnedHostAllocation(false);
        for (size_t i = 0; i < B.GetSize(); ++i) B[i] = 0.5 * static_cast<double>(i);
        C(0) = 1.0, C(1) = 2.0, C(2) = 3.0;
        auto step = [&]() {
            TE("A_e_i = B_e_i C_i", A, B, C);
            TE("B_e_i = A_e_i", B, A);
        };
        step();  // once eagerly: kernels loaded, tensors resident
        hip::BeginCapture();
        step();
        hip::Graph *sequence = hip::EndCapture();
        for (int rep = 0; rep < 3; ++rep) hip::Launch(sequence);
        B.MoveFromGPU();
        // four applications of B_e_i *= C_i in total: one eager, three replays (recording executes nothing)
        CHECK(B(63, 0) == 0.5 * 189 && B(63, 1) == 0.5 * 190 * 16.0 && B(63, 2) == 0.5 * 191 * 81.0);
        bool refused = false;
        Tensor H(64, 3);  // still on the host: using it while recording would need a copy
        hip::BeginCapture();
        try
        {
            TE("A_e_i = B_e_i", A, H);
        }
        catch (const std::runtime_error &)
        {
            refused = true;
        }
        hip::AbortCapture();
        CHECK(refused && !hip::Capturing());
        hip::Destroy(sequence);
    }
}

int main(int argc, char **argv)
{
    const bool gpu = argc > 1 && std::strcmp(argv[1], "gpu") == 0;
    try
    {
        hostTests();
        if (gpu) gpuTests();
    }
    catch (const std::exception &ex)
    {
        std::printf("UNEXPECTED EXCEPTION: %s\n", ex.what());
        return 2;
    }
    std::printf("%d checks, %d failures\n", g_checks, g_failures);
    return g_failures == 0 ? 0 : 1;
}
