// acro::SliceTensor — a view of the trailing dimensions of a parent tensor at fixed leading indices.
// Shares the parent's host and device storage and forwards every residency call to it
// (behaviour of the reference's tensor/SliceTensor.hpp:14-58, tensor/SliceTensor.cpp:142-232).
#ifndef ACRO_HIP_SLICETENSOR_HPP
#define ACRO_HIP_SLICETENSOR_HPP

#include "Tensor.hpp"

namespace acro
{

class SliceTensor : public Tensor
{
  public:
    SliceTensor() : FullT(nullptr), Offset(0) {}
    SliceTensor(Tensor &T, const std::vector<int> &sind) : SliceTensor() { SliceInit(T, sind); }
    template <typename... I>
    SliceTensor(Tensor &T, int d0, I... rest) : SliceTensor()
    {
        SliceInit(T, std::vector<int>{d0, static_cast<int>(rest)...});
    }

    void SliceInit(Tensor &T, const std::vector<int> &sind);
    template <typename... I>
    void SliceInit(Tensor &T, int d0, I... rest)
    {
        SliceInit(T, std::vector<int>{d0, static_cast<int>(rest)...});
    }

    void Retarget(double *, double * = nullptr) override
    {
        ACROBATIC_ASSERT(false, "Retarget not supported on SliceTensors");
    }

    double *GetData() const override;
    double *GetDeviceData() const override;
    void MapToGPU() override;
    void MoveToGPU() override;
    void SwitchToGPU() override;
    void UnmapFromGPU() override;
    void MoveFromGPU() override;
    void SwitchFromGPU() override;
    bool IsMappedToGPU() const override;
    bool IsOnGPU() const override;
    bool IsTransient() const override;

    Tensor *GetParent() const { return FullT; }
    size_t GetOffset() const { return Offset; }

  private:
    Tensor *FullT;
    size_t Offset;
};

}  // namespace acro

#endif
