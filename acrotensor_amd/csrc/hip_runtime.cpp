// Device memory and stream layer: the only place that owns a stream, allocates, copies and checks HIP errors.
// Replaces the reference's util/CudaUtil.hpp:59-108 (error macros, context) and the cudaMalloc/cudaMemcpy/cudaFree
// call sites of tensor/Tensor.cpp:370-428.
#include <hip/hip_runtime.h>

#include <iostream>
#include <mutex>

#include "HipRuntime.hpp"

namespace acro
{

bool isHipReady()
{
    int n = 0;
    hipError_t err = hipGetDeviceCount(&n);
    if (err != hipSuccess)
    {
        (void)hipGetLastError();  // clear the sticky "no device" state
        return false;
    }
    return n > 0;
}

namespace hip
{

void Check(int code, const char *file, int line)
{
    if (code == static_cast<int>(hipSuccess)) return;
    std::string msg = std::string("HIP error: ") + hipGetErrorString(static_cast<hipError_t>(code));
    std::cerr << file << ":" << line << "  " << msg << std::endl;
    ::acro::detail::fail(file, line, msg);
}

namespace
{
std::mutex g_lock;
hipStream_t g_own_stream = nullptr;
hipStream_t g_adopted_stream = nullptr;
bool g_have_info = false;
DeviceInfo g_info;
bool g_capturing = false;

thread_local double *t_no_alloc_scratch = nullptr;
thread_local size_t t_no_alloc_doubles = 0;
thread_local bool t_no_alloc = false;

void notWithoutAllocation(const char *what)
{
    ACROBATIC_ASSERT(!t_no_alloc, std::string(what) +
                                      " is not possible in a call that must not allocate: make the tensors resident "
                                      "and run the same operation once through the ordinary entry point before.");
}

void notWhileCapturing(const char *what)
{
    ACROBATIC_ASSERT(!g_capturing, std::string(what) +
                                       " is not possible while a launch sequence is being recorded: make the tensors "
                                       "resident and run the sequence once before recording it.");
}
}  // namespace

struct Graph
{
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

void *Stream()
{
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_adopted_stream != nullptr) return g_adopted_stream;
    if (g_own_stream == nullptr)
    {
        ACRO_HIP_CHECK(hipStreamCreateWithFlags(&g_own_stream, hipStreamNonBlocking));
    }
    return g_own_stream;
}

void SetStream(void *hip_stream)
{
    notWhileCapturing("Changing the stream");
    hipStream_t incoming = static_cast<hipStream_t>(hip_stream);
    hipStream_t outgoing = static_cast<hipStream_t>(Stream());
    if (incoming == nullptr)
    {
        // back to the library's own stream, created here if it never was
        std::lock_guard<std::mutex> guard(g_lock);
        if (g_own_stream == nullptr) ACRO_HIP_CHECK(hipStreamCreateWithFlags(&g_own_stream, hipStreamNonBlocking));
        incoming = g_own_stream;
    }
    if (incoming != outgoing)
    {
        // Everything already queued on the outgoing stream (kernels, fills, a launched recorded sequence) is made
        // to precede whatever is queued on the incoming stream from now on: tensors written before the switch may
        // be read right after it.  The host does not wait.
        hipEvent_t handover = nullptr;
        ACRO_HIP_CHECK(hipEventCreateWithFlags(&handover, hipEventDisableTiming));
        hipError_t err = hipEventRecord(handover, outgoing);
        if (err == hipSuccess) err = hipStreamWaitEvent(incoming, handover, 0);
        (void)hipEventDestroy(handover);  // released by the runtime once the event has completed
        if (err != hipSuccess)
        {
            // The hand-over failed (an adopted stream that its owner has destroyed already, say).  The switch is made
            // all the same, so that the library does not stay bound to a stream it cannot use, and the failure is
            // reported: work queued before the switch is then NOT ordered before what follows.
            (void)hipGetLastError();
            std::lock_guard<std::mutex> guard(g_lock);
            g_adopted_stream = (incoming == g_own_stream) ? nullptr : incoming;
            throw_error(std::string("Changing the stream: the outgoing stream could not be ordered before the incoming one (") +
                        hipGetErrorString(err) + "); the switch has been made without that ordering.");
        }
    }
    std::lock_guard<std::mutex> guard(g_lock);
    g_adopted_stream = (incoming == g_own_stream) ? nullptr : incoming;
}

void Synchronize()
{
    notWhileCapturing("Synchronising");
    ACRO_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(Stream())));
}

void *Malloc(size_t bytes)
{
    notWithoutAllocation("Allocating device memory");
    notWhileCapturing("Allocating device memory");
    void *p = nullptr;
    ACRO_HIP_CHECK(hipMalloc(&p, bytes));
    return p;
}

void Free(void *dptr)
{
    if (dptr == nullptr) return;
    // Work that still uses the buffer may be queued on the stream (no wait is possible while a sequence is being
    // recorded; this is reached from destructors and must not throw then).
    if (!g_capturing) ACRO_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(Stream())));
    ACRO_HIP_CHECK(hipFree(dptr));
}

void *HostMalloc(size_t bytes)
{
    notWithoutAllocation("Allocating page-locked host memory");
    void *p = nullptr;
    ACRO_HIP_CHECK(hipHostMalloc(&p, bytes, hipHostMallocDefault));
    return p;
}

void HostFree(void *hptr)
{
    if (hptr == nullptr) return;
    if (!g_capturing) ACRO_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(Stream())));
    ACRO_HIP_CHECK(hipHostFree(hptr));
}

NoAllocation::NoAllocation(double *scratch, size_t doubles)
{
    ACROBATIC_ASSERT(!t_no_alloc, "Calls that must not allocate do not nest.");
    t_no_alloc = true;
    t_no_alloc_scratch = scratch;
    t_no_alloc_doubles = doubles;
}

NoAllocation::~NoAllocation()
{
    t_no_alloc = false;
    t_no_alloc_scratch = nullptr;
    t_no_alloc_doubles = 0;
}

bool NoAllocation::Active()
{
    return t_no_alloc;
}

double *NoAllocation::Scratch(size_t doubles)
{
    ACROBATIC_ASSERT(t_no_alloc, "Internal error: no provided scratch buffer outside a call that must not allocate.");
    ACROBATIC_ASSERT(doubles <= t_no_alloc_doubles,
                     "This operation needs " + std::to_string(doubles * sizeof(double)) +
                         " bytes of scratch memory; a call that must not allocate has " +
                         std::to_string(t_no_alloc_doubles * sizeof(double)) + " bytes.  Use the ordinary entry point.");
    return t_no_alloc_scratch;
}

void CopyToDevice(void *dst, const void *src, size_t bytes)
{
    notWhileCapturing("Copying to the device");
    hipStream_t s = static_cast<hipStream_t>(Stream());
    ACRO_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s));
    ACRO_HIP_CHECK(hipStreamSynchronize(s));
}

void CopyToHost(void *dst, const void *src, size_t bytes)
{
    notWhileCapturing("Copying to the host");
    hipStream_t s = static_cast<hipStream_t>(Stream());
    ACRO_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s));
    ACRO_HIP_CHECK(hipStreamSynchronize(s));
}

void BeginCapture()
{
    ACROBATIC_ASSERT(!g_capturing, "A launch sequence is already being recorded.");
    hipStream_t s = static_cast<hipStream_t>(Stream());
    // Relaxed mode: loading the code object of a kernel that is used for the first time inside the recording is
    // not a stream operation and must not invalidate it.
    ACRO_HIP_CHECK(hipStreamBeginCapture(s, hipStreamCaptureModeRelaxed));
    g_capturing = true;
}

Graph *EndCapture()
{
    ACROBATIC_ASSERT(g_capturing, "No launch sequence is being recorded.");
    g_capturing = false;
    hipStream_t s = static_cast<hipStream_t>(Stream());
    Graph *g = new Graph;
    hipError_t err = hipStreamEndCapture(s, &g->graph);
    if (err == hipSuccess) err = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    if (err != hipSuccess)
    {
        if (g->graph != nullptr) (void)hipGraphDestroy(g->graph);
        delete g;
        (void)hipGetLastError();
        ACRO_HIP_CHECK(err);
    }
    return g;
}

void AbortCapture()
{
    if (!g_capturing) return;
    g_capturing = false;
    hipGraph_t discarded = nullptr;
    (void)hipStreamEndCapture(static_cast<hipStream_t>(Stream()), &discarded);
    if (discarded != nullptr) (void)hipGraphDestroy(discarded);
    (void)hipGetLastError();
}

bool Capturing()
{
    return g_capturing;
}

void Launch(Graph *graph)
{
    ACROBATIC_ASSERT(graph != nullptr && graph->exec != nullptr, "Not a recorded launch sequence.");
    notWhileCapturing("Launching a recorded sequence");
    ACRO_HIP_CHECK(hipGraphLaunch(graph->exec, static_cast<hipStream_t>(Stream())));
}

void Destroy(Graph *graph)
{
    if (graph == nullptr) return;
    // A launch of the sequence may still be queued.
    if (!g_capturing) ACRO_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(Stream())));
    if (graph->exec != nullptr) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph != nullptr) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

const DeviceInfo &Info()
{
    std::lock_guard<std::mutex> guard(g_lock);
    if (!g_have_info)
    {
        int dev = 0;
        ACRO_HIP_CHECK(hipGetDevice(&dev));
        hipDeviceProp_t prop;
        ACRO_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
        g_info.num_cus = prop.multiProcessorCount;
        g_info.lds_per_block = prop.sharedMemPerBlock;
        g_info.wavefront = prop.warpSize;
        g_info.arch = prop.gcnArchName;
        g_have_info = true;
    }
    return g_info;
}

}  // namespace hip
}  // namespace acro
