// acro::Tensor — dense row-major fp64 tensor with a host buffer and an optional device mirror.
//
// Public surface follows the reference's tensor/Tensor.hpp:15-126 (constructors taking 1..N dimensions followed
// by optional external host pointer, device pointer and residency flag; Init; operator[] / operator();
// GetRawIndex; Reshape; Retarget; Set; Mult; Print; and the residency calls MapToGPU / MoveToGPU / SwitchToGPU /
// UnmapFromGPU / MoveFromGPU / SwitchFromGPU).  The dimension-list overload families are variadic templates, so
// any rank is accepted, and byte counts are size_t (the reference keeps them in an int, tensor/Tensor.cpp:327).
// The device half calls HIP through HipRuntime.hpp.
#ifndef ACRO_HIP_TENSOR_HPP
#define ACRO_HIP_TENSOR_HPP

#include <cstddef>
#include <type_traits>
#include <vector>
#include "Error.hpp"

namespace acro
{

namespace detail
{
// Collects "d1, d2, ..., [hdata, [ddata, [ongpu]]]" argument tails.
struct TensorArgs
{
    std::vector<int> dims;
    double *hdata = nullptr;
    double *ddata = nullptr;
    bool ongpu = false;
    int nptr = 0;

    void take(bool flag) { ongpu = flag; }
    void take(double *p)
    {
        ACROBATIC_ASSERT(nptr < 2, "Too many data pointers in tensor argument list.");
        (nptr == 0 ? hdata : ddata) = p;
        ++nptr;
    }
    void take(std::nullptr_t) { take(static_cast<double *>(nullptr)); }
    template <typename I, typename = std::enable_if_t<std::is_integral<I>::value && !std::is_same<I, bool>::value>>
    void take(I d)
    {
        ACROBATIC_ASSERT(nptr == 0, "Tensor dimensions must precede the data pointers.");
        dims.push_back(static_cast<int>(d));
    }
    template <typename... A>
    void takeAll(A... a)
    {
        (take(a), ...);
    }
};
}  // namespace detail

class Tensor
{
  public:
    // An empty tensor to be initialised later with Init(...)
    Tensor();
    explicit Tensor(const std::vector<int> &dims, double *hdata = nullptr, double *ddata = nullptr, bool ongpu = false);
    // Tensor(d0, d1, ..., [hdata, [ddata, [ongpu]]])
    template <typename... A>
    explicit Tensor(int d0, A... rest) : Tensor()
    {
        Init(d0, rest...);
    }
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;
    virtual ~Tensor();

    void Init(const std::vector<int> &dims, double *hdata = nullptr, double *ddata = nullptr, bool ongpu = false);
    template <typename... A>
    void Init(int d0, A... rest)
    {
        detail::TensorArgs a;
        a.takeAll(d0, rest...);
        Init(a.dims, a.hdata, a.ddata, a.ongpu);
    }

    // Flat access to the host buffer
    double &operator[](size_t raw_index) { return Data[raw_index]; }
    const double &operator[](size_t raw_index) const { return Data[raw_index]; }

    // Row-major flat index of a multi-index ("most significant index on the left")
    size_t GetRawIndex(const std::vector<int> &indices) const;
    template <typename... I>
    size_t GetRawIndex(int i0, I... rest) const
    {
        const int idx[] = {i0, static_cast<int>(rest)...};
        return RawIndexOf(idx, 1 + static_cast<int>(sizeof...(rest)));
    }

    double &operator()(const std::vector<int> &indices) { return Data[GetRawIndex(indices)]; }
    template <typename... I>
    double &operator()(int i0, I... rest)
    {
        return Data[GetRawIndex(i0, rest...)];
    }

    // New dimensions over the same storage (total size must not change)
    void Reshape(const std::vector<int> &dims);
    template <typename... I>
    void Reshape(int d0, I... rest)
    {
        Reshape(std::vector<int>{d0, static_cast<int>(rest)...});
    }

    int GetRank() const { return static_cast<int>(Dims.size()); }
    // Number of entries.  The reference returns int (tensor/Tensor.hpp:60); a tensor here may hold more than 2^31
    // entries (16 GiB of doubles), so the count is a size_t.
    size_t GetSize() const { return Size; }
    size_t GetByteSize() const { return Size * sizeof(double); }
    int GetDim(int d) const { return Dims[d]; }
    long GetStride(int d) const { return Strides[d]; }   // entries; tensors may exceed 2^31 entries
    const std::vector<int> &GetDims() const { return Dims; }
    virtual double *GetData() const { return Data; }
    virtual double *GetDeviceData() const { return DeviceData; }
    double *GetCurrentData() const { return IsOnGPU() ? GetDeviceData() : GetData(); }

    // Re-point a tensor that wraps externally owned buffers
    virtual void Retarget(double *hdata, double *ddata = nullptr);

    // Residency
    virtual void MapToGPU();       // allocate the device mirror
    virtual void MoveToGPU();      // copy host -> device (mapping first if needed) and mark the device copy current
    virtual void SwitchToGPU();    // mark the device copy current without copying (mapping first if needed)
    virtual void UnmapFromGPU();   // free the device mirror
    virtual void MoveFromGPU();    // copy device -> host if the device copy is current, mark the host copy current
    virtual void SwitchFromGPU();  // mark the host copy current without copying
    virtual bool IsMappedToGPU() const { return MappedToGPU; }
    virtual bool IsOnGPU() const { return OnGPU; }
    virtual bool IsInitialized() const { return Initialized; }

    void Set(double val);  // every entry = val, on whichever side is current
    void Mult(double c);   // every entry *= c, on whichever side is current
    void Print();

    // Extension of the "HIP" policy (no counterpart in the reference): a transient tensor is scratch space of a
    // multi-kernel launch.  When it is produced and consumed inside one fused launch the executor may keep it in
    // on-chip memory only, so its contents in device memory are unspecified afterwards.
    void SetTransient(bool transient) { Transient = transient; }
    virtual bool IsTransient() const { return Transient; }

    // Extension (no counterpart in the reference, which allocates with new[], tensor/Tensor.cpp:196): host buffers
    // that tensors allocate from now on are page-locked, so MoveToGPU / MoveFromGPU run as direct transfers at
    // the rate of the host link instead of through the runtime's staging of pageable memory.  Needs a HIP device.
    static void SetPinnedHostAllocation(bool pinned);
    static bool GetPinnedHostAllocation();

  protected:
    void UpdateStrides();
    void ComputeSize();
    size_t RawIndexOf(const int *idx, int n) const;

    std::vector<int> Dims;
    std::vector<long> Strides;
    size_t Size;

    bool Initialized;
    bool OwnsData;
    bool OwnsDeviceData;  // the device mirror was allocated by MapToGPU (not handed in by the caller)
    bool PinnedData = false;  // the owned host buffer is page-locked
    bool MappedToGPU;
    bool OnGPU;
    bool Transient;
    double *Data;
    double *DeviceData;
};

}  // namespace acro

#endif
