// acro::KernelExecutor — the execution-policy plug-in boundary.  An executor is built for one
// DimensionedMultiKernel and runs it on tensors supplied per call.  Interface as in the reference's
// exec/KernelExecutor.hpp:16-45; the string-keyed factory (exec/KernelExecutor.cpp:106-121) is a registry here,
// so a policy is added by registering a creator instead of editing a switch.
#ifndef ACRO_HIP_KERNEL_EXECUTOR_HPP
#define ACRO_HIP_KERNEL_EXECUTOR_HPP

#include <string>
#include <vector>
#include "DimensionedMultiKernel.hpp"
#include "Tensor.hpp"

namespace acro
{

class IndexMapping;

// An operand of the next launch that need not exist in memory: entry i of `operand` is entry map[i] of `source`
// (a FlatIndexedScatter that the engine recorded in a multi-kernel launch, with a transient result).
struct GatheredInput
{
    Tensor *operand;
    Tensor *source;
    IndexMapping *map;
};

class KernelExecutor
{
  public:
    explicit KernelExecutor(DimensionedMultiKernel *multi_kernel);
    virtual ~KernelExecutor();

    typedef KernelExecutor *(*Creator)(DimensionedMultiKernel *);
    // Policy registry.  "HIP" is registered by the library itself.
    static void Register(const std::string &exec_type, Creator creator);
    static bool IsRegistered(const std::string &exec_type);
    static KernelExecutor *Create(std::string exec_type, DimensionedMultiKernel *multi_kernel);

    virtual std::string GetImplementation() = 0;
    // Implementation that a launch on exactly these tensors would use (policies whose code depends on tensor
    // properties override this; nothing is executed).
    virtual std::string GetImplementation(std::vector<Tensor *> &, std::vector<std::vector<Tensor *>> &)
    {
        return GetImplementation();
    }
    virtual std::string GetExecType() = 0;
    // Applies to the next ExecuteMulti / GetImplementation(tensors) call only.  A policy that cannot read an operand
    // through its map must produce the operand first; the default keeps the list for the sequential fallback below.
    // No counterpart in the reference, whose engine runs a scatter at the call (kernel/TensorEngine.cpp:673-689).
    virtual void SetGatheredInputs(const std::vector<GatheredInput> &gathered) { Gathered = gathered; }
    virtual void ExecuteSingle(Tensor *output, std::vector<Tensor *> &inputs) = 0;
    // Default: one single-kernel executor per kernel, run in order
    virtual void ExecuteMulti(std::vector<Tensor *> &output, std::vector<std::vector<Tensor *>> &inputs);

  protected:
    void MoveTensorsFromGPU(Tensor *output, std::vector<Tensor *> &inputs);
    void MoveTensorsToGPU(Tensor *output, std::vector<Tensor *> &inputs);
    void MoveTensorsToOutputLocation(Tensor *output, std::vector<Tensor *> &inputs);

    std::vector<GatheredInput> Gathered;
    DimensionedMultiKernel *MultiKernel;
    DimensionedKernel *FirstKernel;
    std::vector<DimensionedMultiKernel *> SubKernels;
    std::vector<KernelExecutor *> SubExecutors;
};

}  // namespace acro

#endif
