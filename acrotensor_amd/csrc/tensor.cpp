// Host containers and their device mirrors: Tensor, SliceTensor, IndexVector, IndexMapping.
// Behaviour follows the reference's tensor/Tensor.cpp:166-435, tensor/SliceTensor.cpp:142-232,
// tensor/IndexVector.cpp:14-154 and tensor/IndexMapping.cpp:14-135; device traffic goes through acro::hip.
#include <algorithm>
#include <iostream>
#include <numeric>
#include <vector>

#include "HipRuntime.hpp"
#include "IndexMapping.hpp"
#include "IndexVector.hpp"
#include "SliceTensor.hpp"
#include "Tensor.hpp"

namespace acro
{

// ---------------------------------------------------------------------------------------------- Tensor

namespace
{
bool g_pinned_host_allocation = false;
}

void Tensor::SetPinnedHostAllocation(bool pinned)
{
    ACROBATIC_ASSERT(!pinned || isHipReady(), "Page-locked host memory needs a HIP device.");
    g_pinned_host_allocation = pinned;
}

bool Tensor::GetPinnedHostAllocation()
{
    return g_pinned_host_allocation;
}

Tensor::Tensor()
    : Size(0), Initialized(false), OwnsData(false), OwnsDeviceData(false), MappedToGPU(false), OnGPU(false),
      Transient(false), Data(nullptr), DeviceData(nullptr)
{
}

Tensor::Tensor(const std::vector<int> &dims, double *hdata, double *ddata, bool ongpu) : Tensor()
{
    Init(dims, hdata, ddata, ongpu);
}

void Tensor::Init(const std::vector<int> &dims, double *hdata, double *ddata, bool ongpu)
{
    ACROBATIC_ASSERT(!IsInitialized(), "A tensor can be initialized only once.");
    ACROBATIC_ASSERT(!dims.empty(), "A tensor needs at least one dimension.");
    for (int d : dims)
    {
        ACROBATIC_ASSERT(d > 0, "Every dimension of a tensor must be positive.");
    }
    // External device memory is only accepted next to external host memory, and only a tensor that has a
    // device pointer can start out flagged as resident on the device (reference tensor/Tensor.cpp:189-200).
    ACROBATIC_ASSERT(ddata == nullptr || hdata != nullptr, "A device buffer can only be supplied together with a host buffer (no device-only tensors).");
    ACROBATIC_ASSERT(ddata != nullptr || !ongpu,
                     "External data cannot be flagged as current on the device without a device pointer.");

    Dims = dims;
    UpdateStrides();
    ComputeSize();

    OwnsData = (hdata == nullptr);
    PinnedData = OwnsData && g_pinned_host_allocation;
    if (PinnedData)
        Data = static_cast<double *>(hip::HostMalloc(Size * sizeof(double)));
    else
        Data = OwnsData ? new double[Size] : hdata;
    DeviceData = ddata;
    OwnsDeviceData = false;  // a device buffer handed in stays the caller's
    MappedToGPU = (ddata != nullptr);
    OnGPU = ongpu;
    Initialized = true;
}

Tensor::~Tensor()
{
    // Host and device buffers are released by whoever allocated them, independently of each other: a tensor over a
    // caller's host buffer still owns the device mirror that MapToGPU allocated for it (the reference frees the
    // mirror only together with an owned host buffer, tensor/Tensor.cpp:205-215, and leaks it otherwise).
    if (OwnsData && PinnedData)
    {
        try
        {
            hip::HostFree(Data);
        }
        catch (...)
        {
        }
    }
    else if (OwnsData)
    {
        delete[] Data;
    }
    if (OwnsDeviceData && DeviceData != nullptr)
    {
        try
        {
            hip::Free(DeviceData);
        }
        catch (...)
        {
        }
    }
}

void Tensor::UpdateStrides()
{
    Strides.assign(Dims.size(), 1);
    for (int d = static_cast<int>(Dims.size()) - 2; d >= 0; --d)
    {
        Strides[d] = Strides[d + 1] * Dims[d + 1];
    }
}

void Tensor::ComputeSize()
{
    Size = 1;
    for (int d : Dims) Size *= static_cast<size_t>(d);
}

size_t Tensor::RawIndexOf(const int *idx, int n) const
{
    size_t raw = 0;
    for (int d = 0; d < n; ++d) raw += static_cast<size_t>(idx[d]) * static_cast<size_t>(Strides[d]);
    return raw;
}

size_t Tensor::GetRawIndex(const std::vector<int> &indices) const
{
    return RawIndexOf(indices.data(), static_cast<int>(indices.size()));
}

void Tensor::Reshape(const std::vector<int> &dims)
{
    ACROBATIC_ASSERT(!dims.empty());
    size_t new_size = 1;
    for (int d : dims)
    {
        ACROBATIC_ASSERT(d > 0);
        new_size *= static_cast<size_t>(d);
    }
    ACROBATIC_ASSERT(new_size == Size);
    Dims = dims;
    UpdateStrides();
}

void Tensor::Retarget(double *hdata, double *ddata)
{
    ACROBATIC_ASSERT(!OwnsData);
    if (OwnsDeviceData && DeviceData != ddata)
    {
        hip::Free(DeviceData);  // the mirror of the buffer that is being left
        OwnsDeviceData = false;
    }
    Data = hdata;
    DeviceData = ddata;
    MappedToGPU = (ddata != nullptr);
    if (!MappedToGPU) OnGPU = false;
}

void Tensor::Set(double val)
{
    if (IsOnGPU())
        hip::FillDouble(GetDeviceData(), val, Size);
    else
        std::fill_n(GetData(), Size, val);
}

void Tensor::Mult(double c)
{
    if (IsOnGPU())
    {
        hip::ScaleDouble(GetDeviceData(), c, Size);
    }
    else
    {
        double *p = GetData();
        for (size_t i = 0; i < Size; ++i) p[i] *= c;
    }
}

void Tensor::MapToGPU()
{
    ACROBATIC_ASSERT(!IsMappedToGPU(), "The data already has a device mirror.");
    DeviceData = static_cast<double *>(hip::Malloc(GetByteSize()));
    OwnsDeviceData = true;
    MappedToGPU = true;
}

void Tensor::MoveToGPU()
{
    if (!IsMappedToGPU()) MapToGPU();
    if (!IsOnGPU())
    {
        hip::CopyToDevice(DeviceData, Data, GetByteSize());
        OnGPU = true;
    }
}

void Tensor::SwitchToGPU()
{
    if (!IsMappedToGPU()) MapToGPU();
    OnGPU = true;
}

void Tensor::UnmapFromGPU()
{
    ACROBATIC_ASSERT(IsMappedToGPU(), "There is no device mirror to release.");
    if (OwnsDeviceData) hip::Free(DeviceData);  // a caller's device buffer is only let go of
    OwnsDeviceData = false;
    DeviceData = nullptr;
    MappedToGPU = false;
    OnGPU = false;
}

void Tensor::MoveFromGPU()
{
    if (IsOnGPU())
    {
        hip::CopyToHost(Data, DeviceData, GetByteSize());
        OnGPU = false;
    }
}

void Tensor::SwitchFromGPU()
{
    OnGPU = false;
}

void Tensor::Print()
{
    std::cout << "Dims:  ";
    for (int d : Dims) std::cout << d << "  ";
    std::cout << "\nStrides:  ";
    for (long s : Strides) std::cout << s << "  ";
    std::cout << "\n";
    const double *p = GetData();
    for (size_t i = 0; i < Size; ++i) std::cout << p[i] << "\n";
    std::cout << std::endl;
}

// ----------------------------------------------------------------------------------------- SliceTensor

void SliceTensor::SliceInit(Tensor &T, const std::vector<int> &sind)
{
    ACROBATIC_ASSERT(T.IsInitialized(), "The tensor to slice is not initialized.");
    ACROBATIC_ASSERT(T.GetRank() > static_cast<int>(sind.size()), "Can't slice more dimensions than the tensor rank.");
    ACROBATIC_ASSERT(!sind.empty(), "Can't slice without any leading indices.");
    for (size_t d = 0; d < sind.size(); ++d)
    {
        ACROBATIC_ASSERT(sind[d] >= 0 && sind[d] < T.GetDim(static_cast<int>(d)), "Slice index out of range.");
    }
    FullT = &T;
    Offset = T.GetRawIndex(sind);

    std::vector<int> dims(T.GetDims().begin() + sind.size(), T.GetDims().end());
    double *hdata = T.GetData();
    double *ddata = T.GetDeviceData();
    Initialized = false;
    Init(dims, hdata + Offset, ddata ? ddata + Offset : nullptr, T.IsOnGPU());
}

double *SliceTensor::GetData() const
{
    return FullT->GetData() + Offset;
}

double *SliceTensor::GetDeviceData() const
{
    double *base = FullT->GetDeviceData();
    return base ? base + Offset : nullptr;
}

void SliceTensor::MapToGPU()
{
    FullT->MapToGPU();
}

void SliceTensor::MoveToGPU()
{
    FullT->MoveToGPU();
}

void SliceTensor::SwitchToGPU()
{
    FullT->SwitchToGPU();
}

void SliceTensor::UnmapFromGPU()
{
    // The parent owns the mapping; a view never releases it.
}

void SliceTensor::MoveFromGPU()
{
    FullT->MoveFromGPU();
}

void SliceTensor::SwitchFromGPU()
{
    FullT->SwitchFromGPU();
}

bool SliceTensor::IsMappedToGPU() const
{
    return FullT->IsMappedToGPU();
}

bool SliceTensor::IsOnGPU() const
{
    return FullT->IsOnGPU();
}

bool SliceTensor::IsTransient() const
{
    return Transient || FullT->IsTransient();
}

// ----------------------------------------------------------------------------------------- IndexVector

IndexVector::IndexVector()
    : Size(0), Initialized(false), OwnsData(false), OwnsDeviceData(false), MappedToGPU(false), OnGPU(false), Data(nullptr),
      DeviceData(nullptr)
{
}

IndexVector::IndexVector(int dim, int *hdata, int *ddata, bool ongpu) : IndexVector()
{
    Init(dim, hdata, ddata, ongpu);
}

void IndexVector::Init(int dim, int *hdata, int *ddata, bool ongpu)
{
    ACROBATIC_ASSERT(!IsInitialized(), "An index vector can be initialized only once.");
    ACROBATIC_ASSERT(dim > 0, "An index vector needs a positive length.");
    ACROBATIC_ASSERT(ddata == nullptr || hdata != nullptr, "A device buffer can only be supplied together with a host buffer (no device-only index vectors).");
    ACROBATIC_ASSERT(ddata != nullptr || !ongpu,
                     "External data cannot be flagged as current on the device without a device pointer.");
    Size = static_cast<size_t>(dim);
    OwnsData = (hdata == nullptr);
    Data = OwnsData ? new int[Size] : hdata;
    DeviceData = ddata;
    MappedToGPU = (ddata != nullptr);
    OnGPU = ongpu;
    Initialized = true;
}

IndexVector::~IndexVector()
{
    if (OwnsData) delete[] Data;
    if (OwnsDeviceData && DeviceData != nullptr)
    {
        try
        {
            hip::Free(DeviceData);
        }
        catch (...)
        {
        }
    }
}

void IndexVector::Retarget(int *hdata, int *ddata)
{
    ACROBATIC_ASSERT(!OwnsData);
    if (OwnsDeviceData && DeviceData != ddata)
    {
        hip::Free(DeviceData);
        OwnsDeviceData = false;
    }
    Data = hdata;
    DeviceData = ddata;
    MappedToGPU = (ddata != nullptr);
    if (!MappedToGPU) OnGPU = false;
}

void IndexVector::MapToGPU()
{
    ACROBATIC_ASSERT(!IsMappedToGPU(), "The data already has a device mirror.");
    DeviceData = static_cast<int *>(hip::Malloc(Size * sizeof(int)));
    OwnsDeviceData = true;
    MappedToGPU = true;
}

void IndexVector::MoveToGPU()
{
    if (!IsMappedToGPU()) MapToGPU();
    if (!IsOnGPU())
    {
        hip::CopyToDevice(DeviceData, Data, Size * sizeof(int));
        OnGPU = true;
    }
}

void IndexVector::SwitchToGPU()
{
    if (!IsMappedToGPU()) MapToGPU();
    OnGPU = true;
}

void IndexVector::UnmapFromGPU()
{
    ACROBATIC_ASSERT(IsMappedToGPU(), "There is no device mirror to release.");
    if (OwnsDeviceData) hip::Free(DeviceData);
    OwnsDeviceData = false;
    DeviceData = nullptr;
    MappedToGPU = false;
    OnGPU = false;
}

void IndexVector::MoveFromGPU()
{
    if (IsOnGPU())
    {
        hip::CopyToHost(Data, DeviceData, Size * sizeof(int));
        OnGPU = false;
    }
}

void IndexVector::SwitchFromGPU()
{
    OnGPU = false;
}

void IndexVector::Print()
{
    for (size_t i = 0; i < Size; ++i) std::cout << Data[i] << "\n";
    std::cout << std::endl;
}

// ---------------------------------------------------------------------------------------- IndexMapping

IndexMapping::IndexMapping(int domain_size, int range_size)
    : InverseComputed(false), MappedToGPU(false), OnGPU(false), DomainSize(domain_size), RangeSize(range_size),
      M(range_size), InvM(range_size), InvMOff(domain_size + 1)
{
}

IndexVector &IndexMapping::GetInvMap()
{
    ACROBATIC_ASSERT(InverseComputed, "Trying to access inverse mapping before the inverse is computed.");
    return InvM;
}

IndexVector &IndexMapping::GetInvMapOffsets()
{
    ACROBATIC_ASSERT(InverseComputed, "Trying to access inverse mapping offsets before the inverse is computed.");
    return InvMOff;
}

void IndexMapping::ComputeInverse()
{
    ACROBATIC_ASSERT(!InverseComputed, "Can't compute the inverse mapping twice.");
    int *inv = InvM.GetData();
    int *off = InvMOff.GetData();
    const int *map = M.GetData();

    // Row d of the inverse holds the range entries whose image is d, in increasing range order, which makes the
    // compressed-row sum visit contributions in the same order as a sequential scatter-add over the range.  The
    // reference sorts the range stably by image (tensor/IndexMapping.cpp:31-33); counting rows, prefix-summing and
    // filling in range order gives the same rows in linear time (16.8 M entries: seconds -> tens of milliseconds).
    std::fill(off, off + DomainSize + 1, 0);
    for (int i = 0; i < RangeSize; ++i)
    {
        ACROBATIC_ASSERT(map[i] >= 0 && map[i] < DomainSize, "IndexMapping entry outside of the domain.");
        ++off[map[i] + 1];
    }
    for (int d = 0; d < DomainSize; ++d) off[d + 1] += off[d];
    std::vector<int> next(off, off + DomainSize);
    for (int i = 0; i < RangeSize; ++i) inv[next[map[i]]++] = i;

    InverseComputed = true;
    if (OnGPU)
    {
        InvM.SwitchFromGPU();
        InvM.MoveToGPU();
        InvMOff.SwitchFromGPU();
        InvMOff.MoveToGPU();
    }
}

void IndexMapping::MapToGPU()
{
    M.MapToGPU();
    if (InverseComputed)
    {
        InvM.MapToGPU();
        InvMOff.MapToGPU();
    }
    MappedToGPU = true;
}

void IndexMapping::MoveToGPU()
{
    M.MoveToGPU();
    if (InverseComputed)
    {
        InvM.MoveToGPU();
        InvMOff.MoveToGPU();
    }
    OnGPU = true;
}

void IndexMapping::SwitchToGPU()
{
    M.SwitchToGPU();
    if (InverseComputed)
    {
        InvM.SwitchToGPU();
        InvMOff.SwitchToGPU();
    }
    OnGPU = true;
}

void IndexMapping::UnmapFromGPU()
{
    M.UnmapFromGPU();
    if (InverseComputed)
    {
        if (InvM.IsMappedToGPU()) InvM.UnmapFromGPU();
        if (InvMOff.IsMappedToGPU()) InvMOff.UnmapFromGPU();
    }
    MappedToGPU = false;
    OnGPU = false;
}

void IndexMapping::MoveFromGPU()
{
    M.MoveFromGPU();
    if (InverseComputed)
    {
        InvM.MoveFromGPU();
        InvMOff.MoveFromGPU();
    }
    OnGPU = false;
}

void IndexMapping::SwitchFromGPU()
{
    M.SwitchFromGPU();
    if (InverseComputed)
    {
        InvM.SwitchFromGPU();
        InvMOff.SwitchFromGPU();
    }
    OnGPU = false;
}

}  // namespace acro
