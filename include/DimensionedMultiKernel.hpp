// acro::DimensionedMultiKernel — a group of dimensioned kernels that is executed as one unit.  Variables are
// identified by NAME across the group ("unique variables"), the indices that every kernel carries as a
// non-contraction index are the shared outer indices, and the common loop order puts those first (largest extent
// first).  Reference: kernel/DimensionedMultiKernel.hpp:17-132, kernel/DimensionedMultiKernel.cpp:25-135,162-186.
#ifndef ACRO_HIP_DIMENSIONED_MULTI_KERNEL_HPP
#define ACRO_HIP_DIMENSIONED_MULTI_KERNEL_HPP

#include <map>
#include <string>
#include <utility>
#include <vector>
#include "DimensionedKernel.hpp"

namespace acro
{

class DimensionedMultiKernel
{
  public:
    explicit DimensionedMultiKernel(std::vector<DimensionedKernel *> &kernels);
    explicit DimensionedMultiKernel(DimensionedKernel *kernel);

    int GetNumKernels() const { return static_cast<int>(Kernels.size()); }
    int GetNumIndices() const { return static_cast<int>(AllIndexNames.size()); }
    int GetNumOuterIndices() const { return static_cast<int>(SharedOuterIndexNames.size()); }
    int GetNumContractionIndices() const { return static_cast<int>(ContractionIndexNames.size()); }
    int GetNumVars() const { return GetNumInputVars() + GetNumOutputVars(); }
    int GetNumUVars() const { return static_cast<int>(UVariToFirstKiVari.size()); }
    int GetNumInputVars() const;
    int GetNumOutputVars() const { return GetNumKernels(); }

    std::string GetDimensionedNameString() const;
    const std::string &GetLoopIndex(int loopi) const { return LoopIndices[loopi]; }
    int GetIndexLoopNum(const std::string &idx) const;  // -1 when absent
    void SetLoopIndices(const std::vector<std::string> &idx_list);

    // (ki, vari): kernel number and variable number inside it, vari == -1 for that kernel's output
    int GetVarRank(int ki, int vari) const;
    int GetVarDimLoopNum(int ki, int vari, int dim) const;
    int GetLoopNumVarDim(int loop_num, int ki, int vari) const;
    bool IsVarDependentOnLoop(int ki, int vari, int loop_num) const;
    bool IsContractionLoop(int loop_num) const;
    bool IsSharedOuterLoop(int loop_num) const;
    bool IsOutputUVar(int uvari) const;
    bool IsInputUVar(int uvari) const;

    const std::vector<int> &GetLoopDims() const { return LoopDims; }
    int GetLoopDim(int i) const { return LoopDims[i]; }
    int GetLoopDim(const std::string &idx) const { return GetLoopDim(GetIndexLoopNum(idx)); }
    int GetLoopStride(int i) const { return LoopStrides[i]; }

    int GetFlatIdxSize() const;
    int GetSharedOuterIdxSize() const;
    int GetIdxSizeForFirstNumLoops(int num_loops) const;
    int GetVarDimStride(int ki, int vari, int dim) const;
    int GetVarSize(int ki, int vari) const;
    int GetVarSize(int uvari) const;
    int GetVarLoopDepth(int ki, int vari) const;

    int GetUVari(int ki, int vari) const { return KiVariToUVari.at(std::make_pair(ki, vari)); }
    std::pair<int, int> GetFirstKiVariForUVari(int uvari) const { return UVariToFirstKiVari[uvari]; }

    int GetVarStorageReqForInnerLoops(int ki, int vari, int num_loops) const;
    int GetInputStorageReqForInnerLoops(int num_loops) const;
    int GetOutputStorageReqForInnerLoops(int num_loops) const;
    int GetTotalStorageReqForInnerLoops(int num_loops) const;
    int GetIndexSpaceSizeForInnerLoops(int num_loops) const;
    void GetVarIndexOffsetsForInnerLoops(int ki, int vari, int num_inner_loops, std::vector<int> &var_off,
                                         std::vector<int> &loop_off) const;

    std::vector<DimensionedKernel *> Kernels;
    std::vector<std::string> AllIndexNames;
    std::vector<std::string> ContractionIndexNames;
    std::vector<std::string> SharedOuterIndexNames;
    std::vector<std::string> LoopIndices;

  private:
    void InitMKLVars();

    std::map<std::pair<int, int>, int> KiVariToUVari;
    std::vector<std::pair<int, int>> UVariToFirstKiVari;
    std::vector<int> LoopDims;
    std::vector<int> LoopStrides;
};

}  // namespace acro

#endif
