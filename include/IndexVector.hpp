// acro::IndexVector — an int array with the same host/device residency protocol as Tensor
// (reference: tensor/IndexVector.hpp:14-57, tensor/IndexVector.cpp:88-154).
#ifndef ACRO_HIP_INDEXVECTOR_HPP
#define ACRO_HIP_INDEXVECTOR_HPP

#include <cstddef>
#include "Error.hpp"

namespace acro
{

class IndexVector
{
  public:
    IndexVector();
    explicit IndexVector(int dim, int *hdata = nullptr, int *ddata = nullptr, bool ongpu = false);
    IndexVector(const IndexVector &) = delete;
    IndexVector &operator=(const IndexVector &) = delete;
    ~IndexVector();
    void Init(int dim, int *hdata = nullptr, int *ddata = nullptr, bool ongpu = false);

    int GetSize() const { return static_cast<int>(Size); }
    int *GetData() const { return Data; }
    int *GetDeviceData() const { return DeviceData; }
    int *GetCurrentData() const { return OnGPU ? DeviceData : Data; }
    int &operator[](int raw_index) { return Data[raw_index]; }

    void Retarget(int *hdata, int *ddata);

    void MapToGPU();
    void MoveToGPU();
    void SwitchToGPU();
    void UnmapFromGPU();
    void MoveFromGPU();
    void SwitchFromGPU();
    bool IsMappedToGPU() const { return MappedToGPU; }
    bool IsOnGPU() const { return OnGPU; }
    bool IsInitialized() const { return Initialized; }

    void Print();

  private:
    size_t Size;
    bool Initialized;
    bool OwnsData;
    bool OwnsDeviceData;  // the device mirror was allocated by MapToGPU (not handed in by the caller)
    bool MappedToGPU;
    bool OnGPU;
    int *Data;
    int *DeviceData;
};

}  // namespace acro

#endif
