// Device memory and stream layer of the "HIP" policy (replaces the role of the reference's
// util/CudaUtil.hpp:59-108,175-184: error checks, context handling, isCudaReady, and the cudaMalloc /
// cudaMemcpy / cudaFree call sites in tensor/Tensor.cpp:370-428 and tensor/IndexVector.cpp:88-154).
//
// All device work of the library (copies, fills, generated kernels, batched ops) is issued on ONE stream that
// this layer owns, so stream order alone makes producer/consumer sequences correct; only device-to-host
// copies and explicit Synchronize() calls block the host.  Byte counts are size_t throughout.
#ifndef ACRO_HIP_RUNTIME_HPP
#define ACRO_HIP_RUNTIME_HPP

#include <cstddef>
#include <string>
#include "Error.hpp"

namespace acro
{

// True when a HIP device can be used by this process (hipGetDeviceCount > 0).  Never throws.
bool isHipReady();

namespace hip
{
// The stream every operation of the library is enqueued on (a hipStream_t passed as void* so that public
// headers do not need the HIP headers).  Created lazily with default priority; never the null stream.
void *Stream();
// Adopt an externally created stream (the library then never destroys it).  nullptr restores the own stream.
void SetStream(void *hip_stream);
void Synchronize();

void *Malloc(size_t bytes);
void Free(void *dptr);
void *HostMalloc(size_t bytes);   // page-locked host memory
void HostFree(void *hptr);
void CopyToDevice(void *dst, const void *src, size_t bytes);    // returns after the host buffer may be reused
void CopyToHost(void *dst, const void *src, size_t bytes);      // returns after the data has arrived
void FillDouble(double *d, double value, size_t n);             // d[i] = value   (async on Stream())
void ScaleDouble(double *d, double factor, size_t n);           // d[i] *= factor (async on Stream())

// Recorded launch sequences (hipGraph).  Between BeginCapture() and EndCapture() everything the library enqueues on
// Stream() (generated kernels, batched operations, fills) is recorded instead of executed; Launch() then enqueues
// the whole recorded sequence with one call.  The recorded work must not need the host: allocations, host <-> device
// copies and Synchronize() throw while recording, so tensors have to be resident and every kernel of the sequence
// has to have run once before (its code object is then loaded and its scratch buffer allocated).  The reference
// has no counterpart: it launches kernel by kernel on the null stream (exec/CudaExecutor.cpp:70-101).
struct Graph;
void BeginCapture();
Graph *EndCapture();           // ends the recording (also after an error in between) and instantiates it
void AbortCapture();           // ends a recording and discards it; no-op when none is active
bool Capturing();
void Launch(Graph *graph);     // asynchronous, in stream order with everything else on Stream()
void Destroy(Graph *graph);

// Calls that must not allocate.  While a NoAllocation object lives on a thread, that thread's calls into the
// library allocate no device or page-locked memory and load no code object: Malloc, HostMalloc and the first launch
// of a kernel that is not loaded yet throw (Free only ever runs from destructors and is not reached), and launches
// that need a scratch buffer take `doubles` entries at `scratch` (device memory the caller of this layer provides;
// larger requests throw) instead of a buffer of their own.
class NoAllocation
{
  public:
    NoAllocation(double *scratch, size_t doubles);
    ~NoAllocation();
    NoAllocation(const NoAllocation &) = delete;
    NoAllocation &operator=(const NoAllocation &) = delete;
    static bool Active();
    // The provided scratch buffer, after checking that `doubles` entries fit.  Only while Active().
    static double *Scratch(size_t doubles);
};

// Multiprocessor count, LDS bytes per workgroup, wavefront size of the current device (cached).
struct DeviceInfo
{
    int num_cus;
    size_t lds_per_block;
    int wavefront;
    std::string arch;
};
const DeviceInfo &Info();

// Throws std::runtime_error("<file>:  <line>  HIP error: ...") when code != hipSuccess.
void Check(int hip_error_code, const char *file, int line);
}  // namespace hip

}  // namespace acro

#define ACRO_HIP_CHECK(call) ::acro::hip::Check(static_cast<int>(call), __FILE__, __LINE__)

#endif
