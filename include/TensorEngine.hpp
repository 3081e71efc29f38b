// acro::TensorEngine — the user-facing engine: TE("S_i_j = A_n_i_j B_n", S, A, B).
// Public surface follows the reference's kernel/TensorEngine.hpp:26-114 (policy string, call operator for one
// to many input tensors, GetImplementation, Begin/EndMultiKernelLaunch, the five non-contraction operations,
// Clear, IsGPUAvailable).  The input-count overload families are variadic templates.  The execution policy that
// this library provides is "HIP" (drop-in for the reference's "Cuda"); other policy strings are accepted when an
// executor has been registered for them with KernelExecutor::Register.
#ifndef ACRO_HIP_TENSOR_ENGINE_HPP
#define ACRO_HIP_TENSOR_ENGINE_HPP

#include <string>
#include <unordered_map>
#include <vector>
#include "DimensionedMultiKernel.hpp"
#include "HipRuntime.hpp"
#include "IndexMapping.hpp"
#include "KernelExecutor.hpp"
#include "NonContractionOps.hpp"

namespace acro
{

class TensorEngine
{
  public:
    TensorEngine();
    explicit TensorEngine(const char *bare_exec_type);
    explicit TensorEngine(const std::string &exec_type);
    TensorEngine(const TensorEngine &) = delete;
    TensorEngine &operator=(const TensorEngine &) = delete;
    ~TensorEngine();

    void SetExecutorType(const char *bare_exec_type);
    void SetExecutorType(const std::string &exec_type);
    std::string GetExecType() const { return ExecutorType; }

    // TE(kernel, out, in1, in2, ...)
    template <typename... In>
    void operator()(const std::string &kernel_str, Tensor &out, Tensor &in1, In &...more)
    {
        std::vector<Tensor *> inputs = {&in1, &more...};
        (*this)(kernel_str, &out, inputs);
    }
    void operator()(const std::string &kernel_str, Tensor *out, std::vector<Tensor *> &inputs);

    template <typename... In>
    std::string GetImplementation(const std::string &kernel_str, Tensor &out, Tensor &in1, In &...more)
    {
        std::vector<Tensor *> inputs = {&in1, &more...};
        return GetImplementation(kernel_str, &out, inputs);
    }
    std::string GetImplementation(const std::string &kernel_str, Tensor *out, std::vector<Tensor *> &inputs);

    void BatchMatrixInverse(Tensor &Ainv, Tensor &A);
    void BatchMatrixDet(Tensor &Adet, Tensor &A);
    void BatchMatrixInvDet(Tensor &Ainv, Tensor &Adet, Tensor &A);
    void FlatIndexedScatter(Tensor &Aout, Tensor &Ain, IndexMapping &M);
    void FlatIndexedSumGather(Tensor &Aout, Tensor &Ain, IndexMapping &M);

    void Clear();
    bool IsGPUAvailable() { return isHipReady(); }
    // A FlatIndexedScatter issued in between whose result is marked transient and is only read by the kernels that
    // follow is not run at all: those kernels read the source vector through the index map.
    // Kernels issued between Begin and End are captured and executed as ONE fused launch by End.  Batched matrix
    // inverses and determinants issued in between are captured too when a later kernel of the capture reads their
    // result: they become kernels of the fused launch, and a result marked transient never reaches device memory.
    // (The reference runs them at once, kernel/TensorEngine.cpp:627-671; the order of operations is the same.)
    void BeginMultiKernelLaunch();
    void EndMultiKernelLaunch();
    // True between BeginMultiKernelLaunch and EndMultiKernelLaunch: calls are being recorded, not run.
    bool InMultiKernelLaunch() const { return IsMultiKernelLaunch; }

    // Ends a capture started by BeginMultiKernelLaunch WITHOUT executing it and returns the implementation the
    // launch would have used (needs no device).
    std::string EndMultiKernelLaunchGetImplementation();
    // Implementation text of the executor used by the most recent launch ("" before the first one).
    std::string GetLastImplementation();

  private:
    TensorKernel *GetAddTensorKernel(const std::string &kernel_str);
    DimensionedKernel *GetAddDimensionedKernel(TensorKernel *kernel, Tensor *output, std::vector<Tensor *> &inputs);
    KernelExecutor *GetAddKernelExecutor();
    void MoveToComputeLocation(Tensor &T);
    void SwitchToComputeLocation(Tensor &T);
    void MoveToComputeLocation(IndexMapping &M);
    void ResetCapture();
    // A batched matrix operation recorded inside a multi-kernel launch, ahead of captured kernel number `position`.
    struct RecordedMatrixOp
    {
        size_t position;
        Tensor *inverse;      // null for a determinant alone
        Tensor *determinant;  // null for an inverse alone
        Tensor *matrices;
        // a recorded FlatIndexedScatter or FlatIndexedSumGather instead (the three above are null then)
        Tensor *scatter_out;
        Tensor *scatter_in;
        IndexMapping *map;
        bool sum_gather = false;  // scatter_out / scatter_in are the sum-gather's result and operand
    };
    // Executes the capture (or, with `implementation` set, only describes it).
    void FinishCapture(std::string *implementation);
    bool MatrixOpAsKernels(const RecordedMatrixOp &op, const std::vector<DimensionedKernel *> &kernels,
                           const std::vector<Tensor *> &outputs, const std::vector<std::vector<Tensor *>> &inputs,
                           std::vector<DimensionedKernel *> &op_kernels, std::vector<Tensor *> &op_outputs,
                           std::vector<std::vector<Tensor *>> &op_inputs);
    TensorKernel *GetAddTensorKernel(const std::string &kernel_str, const std::string &function);

    std::string ExecutorType;
    std::unordered_map<std::string, TensorKernel *> KernelMap;
    std::unordered_map<std::string, DimensionedKernel *> DimensionedKernelMap;
    std::unordered_map<std::string, KernelExecutor *> ExecutorMap;
    std::vector<DimensionedMultiKernel *> OwnedMultiKernels;
    // What the previous call with the same kernel string / the previous capture resolved to: a repeated call with the
    // same extents (the usual case inside a solver's loop) skips building and hashing the name strings.
    struct DimensionedMemo
    {
        std::vector<int> dims;  // rank and extents of the output and of every input
        DimensionedKernel *kernel = nullptr;
    };
    std::unordered_map<const TensorKernel *, DimensionedMemo> LastDimensioned;
    std::vector<int> DimsOfThisCall;
    std::vector<DimensionedKernel *> LastCapture;
    KernelExecutor *LastCaptureExecutor = nullptr;
    std::string ComputeLocation;
    NonContractionOps *Ops;

    bool IsMultiKernelLaunch;
    std::vector<DimensionedKernel *> MKLKernels;
    std::vector<Tensor *> MKLOutputT;
    std::vector<std::vector<Tensor *>> MKLInputT;
    std::vector<RecordedMatrixOp> MKLMatrixOps;
    KernelExecutor *LastExecutor;
};

}  // namespace acro

#endif
