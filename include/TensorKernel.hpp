// acro::TensorKernel — the parsed form of an Einstein-notation kernel string such as
// "S_i_j = A_n_i_j B_n".  Grammar, index ordering and name mangling follow the reference's
// kernel/TensorKernel.hpp:25-113 and kernel/TensorKernel.cpp:26-139,327-403:
//
//   kernel := var eqop var+          eqop := "=" | "+=" | "-="
//   var    := NAME ("_" IDX)+        NAME := [A-Z][A-Za-z0-9]*      IDX := [a-z0-9]+
//
// White space is removed before parsing.  AllIndexNames lists the output indices first, then every index that
// only appears on the right-hand side (a contraction index) in order of first appearance.
#ifndef ACRO_HIP_TENSOR_KERNEL_HPP
#define ACRO_HIP_TENSOR_KERNEL_HPP

#include <string>
#include <vector>
#include "Tensor.hpp"

namespace acro
{

class KernelVar
{
  public:
    std::string Name;
    std::vector<std::string> IndexNames;
    std::vector<int> LoopNums;  // for each tensor dimension, the position of its index in LoopIndices
};

class TensorKernel
{
  protected:
    TensorKernel() {}

  public:
    explicit TensorKernel(const char *kernel);
    explicit TensorKernel(const std::string &kernel);
    // A kernel whose right-hand side is not a product but a function of its single operand's trailing matrix
    // (see Function below).  Used by the engine for batched matrix operations recorded in a multi-kernel launch.
    TensorKernel(const std::string &kernel, const std::string &function);
    virtual ~TensorKernel() {}

    int GetNumIndices() const { return static_cast<int>(AllIndexNames.size()); }
    int GetNumOuterIndices() const { return GetNumIndices() - GetNumContractionIndices(); }
    int GetNumContractionIndices() const { return static_cast<int>(ContractionIndexNames.size()); }
    int GetNumVars() const { return GetNumInputVars() + 1; }
    int GetNumInputVars() const { return static_cast<int>(InputVars.size()); }

    // vari == -1 names the output variable in all of the following
    int GetVarRank(int vari) const;
    const std::string &GetLoopIndex(int loopi) const { return LoopIndices[loopi]; }
    int GetLoopNum(const std::string &idx) const;
    virtual void SetLoopIndices(const std::vector<std::string> &idx_list);
    int GetVarDimLoopNum(int vari, int dim) const;
    int GetLoopNumVarDim(int loop_num, int vari) const;  // -1 when the variable does not carry that loop index
    bool IsVarDependentOnLoop(int vari, int loop_num) const;
    bool IsDependentOnIndex(const std::string &idx) const;
    bool IsDependentOnLoop(int loop_num) const;
    bool IsContractionIndex(const std::string &idx) const;
    bool IsContractionLoop(int loop_num) const;
    bool IsContractionVar(int vari) const;
    int GetLoopDepth() const;
    int GetVarLoopDepth(int vari) const;
    const std::string &GetVarName(int vari) const;
    const KernelVar &GetVar(int vari) const { return vari < 0 ? OutputVar : InputVars[vari]; }

    // "Out_i_j" + ("eq" | "pe" | "me") + "In1_..." "In2_..."
    std::string GetNameString() const;
    // GetNameString() + "_" + "_<dim>" for every loop index
    virtual std::string GetDimensionedNameString()
    {
        ACROBATIC_ASSERT(false);
        return "";
    }
    virtual std::string GetDimensionedNameString(Tensor *output, std::vector<Tensor *> &inputs);
    // Extent of every loop index taken from the tensors; throws when two uses of an index disagree
    std::vector<int> GetLoopIdxSizes(Tensor *output, std::vector<Tensor *> &inputs) const;

    std::string KernelStr;
    // "" for a contraction.  "inv": "Ainv_..._m_n = A_..._m_n" writes, for every leading index, the inverse of the
    // trailing m x n matrix (m = n <= 3) laid out as the reference's batched inverse lays it out
    // (ops/NativeCPUOps.hpp:38-67).  "det": "Adet_... = A_..._m_n" writes its determinant (ops/NativeCPUOps.hpp:70-86).
    // The reference has no such kernels: its engine runs these operations outside the kernel machinery
    // (kernel/TensorEngine.cpp:627-671).
    std::string Function;
    KernelVar OutputVar;
    std::string EqOperator;
    std::vector<KernelVar> InputVars;
    std::vector<std::string> AllIndexNames;
    std::vector<std::string> ContractionIndexNames;
    std::vector<std::string> LoopIndices;

  private:
    void ParseKernel();
    void SetVarLoopNums();
};

}  // namespace acro

#endif
