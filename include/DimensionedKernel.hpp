// acro::DimensionedKernel — a TensorKernel bound to tensor shapes: every loop index has an extent and a stride
// in the flattened loop space.  Reference: kernel/DimensionedKernel.hpp:17-73, kernel/DimensionedKernel.cpp.
#ifndef ACRO_HIP_DIMENSIONED_KERNEL_HPP
#define ACRO_HIP_DIMENSIONED_KERNEL_HPP

#include <string>
#include <vector>
#include "TensorKernel.hpp"

namespace acro
{

class DimensionedKernel : public TensorKernel
{
  public:
    DimensionedKernel(TensorKernel *kernel, Tensor *output, std::vector<Tensor *> &inputs);

    const std::vector<int> &GetLoopDims() const { return LoopDims; }
    const std::vector<int> &GetLoopStrides() const { return LoopStrides; }
    int GetLoopDim(const std::string &idx) const { return LoopDims[GetLoopNum(idx)]; }
    int GetLoopStride(const std::string &idx) const { return LoopStrides[GetLoopNum(idx)]; }
    int GetLoopDim(int i) const { return LoopDims[i]; }
    int GetLoopStride(int i) const { return LoopStrides[i]; }
    // Permute the loops; an index this kernel does not use becomes a loop of extent 1
    void SetLoopIndices(const std::vector<std::string> &idx_list) override;

    // "__dim_<d>..." in AllIndexNames order
    std::string GetLoopDimsString() const;
    std::string GetDimensionedNameString() override { return GetNameString() + GetLoopDimsString(); }
    std::string GetDimensionedNameString(Tensor *, std::vector<Tensor *> &) override
    {
        return GetDimensionedNameString();
    }

    int GetFlatIdxSize() const;  // product of all loop extents
    int GetOutIdxSize() const;   // product of the non-contraction loop extents
    int GetContIdxSize() const;  // product of the contraction loop extents
    int GetIdxSizeForFirstNumLoops(int num_loops) const;
    int GetLoopsIdxSize(const std::vector<int> &loops) const;

    int GetVarDimSize(int vari, int dim) const { return LoopDims[GetVarDimLoopNum(vari, dim)]; }
    int GetVarDimStride(int vari, int dim) const;  // row-major stride of a variable's dimension
    int GetVarSize(int vari) const;                // number of entries of a variable

    int GetVarStorageReqForInnerLoops(int vari, int num_loops) const;
    int GetInputStorageReqForInnerLoops(int num_loops) const;
    int GetOutputStorageReqForInnerLoops(int num_loops) const;
    int GetTotalStorageReqForInnerLoops(int num_loops) const;
    int GetIndexSpaceSizeForInnerLoops(int num_loops) const;
    void GetVarIndexOffsetsForInnerLoops(int vari, int num_inner_loops, std::vector<int> &var_off,
                                         std::vector<int> &loop_off) const;

  private:
    void RecomputeStrides();
    std::vector<int> LoopDims;
    std::vector<int> LoopStrides;
};

}  // namespace acro

#endif
