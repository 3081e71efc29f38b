// extern "C" boundary of the library: flattens the C++ API (TensorEngine, Tensor, SliceTensor, IndexMapping) into
// plain-pointer entry points and converts exceptions into error codes + a per-thread message.
#include <hip/hip_runtime.h>

#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>

#include "AcroTensor.hpp"
#include "acrotensor_hip.h"
#include "hip_kernel.hpp"

using namespace acro;

struct acro_tensor
{
    Tensor *t;
};
struct acro_engine
{
    TensorEngine te;
};
struct acro_index_mapping
{
    IndexMapping *m;
};

namespace
{

thread_local std::string g_last_error;

template <typename F>
int guarded(F &&body)
{
    try
    {
        body();
        g_last_error.clear();
        return 0;
    }
    catch (const std::exception &ex)
    {
        g_last_error = ex.what();
        return 1;
    }
    catch (...)
    {
        g_last_error = "unknown exception";
        return 2;
    }
}

void require(bool cond, const char *msg)
{
    if (!cond) throw_error(msg);
}

}  // namespace

static void resolveNoAllocScratch();  // defined with the scratch array below

namespace
{

void copyOut(const std::string &s, char *buf, size_t buflen, size_t *needed)
{
    if (needed != nullptr) *needed = s.size() + 1;
    if (buf != nullptr && buflen > 0)
    {
        size_t n = s.size() < buflen - 1 ? s.size() : buflen - 1;
        std::memcpy(buf, s.data(), n);
        buf[n] = '\0';
    }
}

std::vector<Tensor *> unwrap(acro_tensor *const *list, int n)
{
    require(n >= 0 && (n == 0 || list != nullptr), "null tensor list");
    std::vector<Tensor *> v(n);
    for (int i = 0; i < n; ++i)
    {
        require(list[i] != nullptr, "null tensor handle");
        v[i] = list[i]->t;
    }
    return v;
}

std::string jsonList(const std::vector<std::string> &v)
{
    std::string s = "[";
    for (size_t i = 0; i < v.size(); ++i) s += (i ? ",\"" : "\"") + v[i] + "\"";
    return s + "]";
}

std::string jsonList(const std::vector<int> &v)
{
    std::string s = "[";
    for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + std::to_string(v[i]);
    return s + "]";
}

}  // namespace

extern "C" {

const char *acro_last_error(void)
{
    return g_last_error.c_str();
}

int acro_hip_is_ready(void)
{
    return isHipReady() ? 1 : 0;
}

int acro_hip_synchronize(void)
{
    return guarded([] { hip::Synchronize(); });
}

int acro_hip_set_stream(void *hip_stream)
{
    return guarded([&] { hip::SetStream(hip_stream); });
}

void *acro_hip_get_stream(void)
{
    void *s = nullptr;
    guarded([&] { s = hip::Stream(); });
    return s;
}

int acro_hip_event_create(void **event)
{
    return guarded([&] {
        require(event != nullptr, "null event pointer");
        hipEvent_t ev;
        ACRO_HIP_CHECK(hipEventCreate(&ev));
        *event = ev;
    });
}

int acro_hip_event_record(void *event)
{
    return guarded([&] {
        require(!hip::Capturing(), "events cannot be recorded while a launch sequence is being recorded");
        ACRO_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(hip::Stream())));
    });
}

int acro_hip_event_elapsed_ms(void *start, void *stop, float *ms)
{
    return guarded([&] {
        require(ms != nullptr, "null result pointer");
        ACRO_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
        ACRO_HIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    });
}

int acro_hip_event_destroy(void *event)
{
    return guarded([&] { ACRO_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event))); });
}

int acro_hip_graph_begin_capture(void)
{
    return guarded([] { hip::BeginCapture(); });
}

int acro_hip_graph_end_capture(acro_hip_graph **out)
{
    return guarded([&] {
        require(out != nullptr, "null graph pointer");
        *out = reinterpret_cast<acro_hip_graph *>(hip::EndCapture());
    });
}

int acro_hip_graph_abort_capture(void)
{
    return guarded([] { hip::AbortCapture(); });
}

int acro_hip_graph_launch(acro_hip_graph *g)
{
    return guarded([&] { hip::Launch(reinterpret_cast<hip::Graph *>(g)); });
}

int acro_hip_graph_destroy(acro_hip_graph *g)
{
    return guarded([&] { hip::Destroy(reinterpret_cast<hip::Graph *>(g)); });
}

// ------------------------------------------------------------------------------------------------ tensor

int acro_tensor_set_pinned_host_allocation(int pinned)
{
    return guarded([&] { Tensor::SetPinnedHostAllocation(pinned != 0); });
}

int acro_tensor_create(int rank, const int *dims, double *hdata, double *ddata, int ongpu, acro_tensor **out)
{
    return guarded([&] {
        require(out != nullptr, "null output handle");
        require(rank >= 0 && (rank == 0 || dims != nullptr), "null dims");
        std::vector<int> d(dims, dims + rank);
        Tensor *t = new Tensor();
        try
        {
            t->Init(d, hdata, ddata, ongpu != 0);
        }
        catch (...)
        {
            delete t;
            throw;
        }
        *out = new acro_tensor{t};
    });
}

int acro_tensor_create_slice(acro_tensor *parent, int num_indices, const int *indices, acro_tensor **out)
{
    return guarded([&] {
        require(out != nullptr && parent != nullptr, "null handle");
        require(num_indices >= 0 && (num_indices == 0 || indices != nullptr), "null slice indices");
        std::vector<int> idx(indices, indices + num_indices);
        SliceTensor *s = new SliceTensor();
        try
        {
            s->SliceInit(*parent->t, idx);
        }
        catch (...)
        {
            delete s;
            throw;
        }
        *out = new acro_tensor{s};
    });
}

int acro_tensor_destroy(acro_tensor *t)
{
    return guarded([&] {
        if (t == nullptr) return;
        delete t->t;
        delete t;
    });
}

int acro_tensor_rank(const acro_tensor *t) { return t ? t->t->GetRank() : -1; }
long long acro_tensor_size(const acro_tensor *t) { return t ? static_cast<long long>(t->t->GetSize()) : -1; }
int acro_tensor_dim(const acro_tensor *t, int d) { return (t && d >= 0 && d < t->t->GetRank()) ? t->t->GetDim(d) : -1; }
long long acro_tensor_stride(const acro_tensor *t, int d)
{
    return (t && d >= 0 && d < t->t->GetRank()) ? t->t->GetStride(d) : -1;
}
double *acro_tensor_data(const acro_tensor *t) { return t ? t->t->GetData() : nullptr; }
double *acro_tensor_device_data(const acro_tensor *t) { return t ? t->t->GetDeviceData() : nullptr; }

int acro_tensor_reshape(acro_tensor *t, int rank, const int *dims)
{
    return guarded([&] {
        require(t != nullptr && dims != nullptr, "null handle");
        t->t->Reshape(std::vector<int>(dims, dims + rank));
    });
}

int acro_tensor_retarget(acro_tensor *t, double *hdata, double *ddata)
{
    return guarded([&] {
        require(t != nullptr, "null handle");
        t->t->Retarget(hdata, ddata);
    });
}

#define ACRO_TENSOR_CALL(cname, method)             \
    int cname(acro_tensor *t)                       \
    {                                               \
        return guarded([&] {                        \
            require(t != nullptr, "null handle");   \
            t->t->method();                         \
        });                                         \
    }
ACRO_TENSOR_CALL(acro_tensor_map_to_gpu, MapToGPU)
ACRO_TENSOR_CALL(acro_tensor_move_to_gpu, MoveToGPU)
ACRO_TENSOR_CALL(acro_tensor_switch_to_gpu, SwitchToGPU)
ACRO_TENSOR_CALL(acro_tensor_unmap_from_gpu, UnmapFromGPU)
ACRO_TENSOR_CALL(acro_tensor_move_from_gpu, MoveFromGPU)
ACRO_TENSOR_CALL(acro_tensor_switch_from_gpu, SwitchFromGPU)
#undef ACRO_TENSOR_CALL

int acro_tensor_is_mapped_to_gpu(const acro_tensor *t) { return (t && t->t->IsMappedToGPU()) ? 1 : 0; }
int acro_tensor_is_on_gpu(const acro_tensor *t) { return (t && t->t->IsOnGPU()) ? 1 : 0; }

int acro_tensor_set(acro_tensor *t, double value)
{
    return guarded([&] {
        require(t != nullptr, "null handle");
        t->t->Set(value);
    });
}

int acro_tensor_mult(acro_tensor *t, double factor)
{
    return guarded([&] {
        require(t != nullptr, "null handle");
        t->t->Mult(factor);
    });
}

int acro_tensor_set_transient(acro_tensor *t, int transient)
{
    return guarded([&] {
        require(t != nullptr, "null handle");
        t->t->SetTransient(transient != 0);
    });
}

// ----------------------------------------------------------------------------------------- index mapping

int acro_index_mapping_create(int domain_size, int range_size, acro_index_mapping **out)
{
    return guarded([&] {
        require(out != nullptr, "null output handle");
        require(domain_size > 0 && range_size > 0, "IndexMapping sizes must be positive");
        *out = new acro_index_mapping{new IndexMapping(domain_size, range_size)};
    });
}

int acro_index_mapping_destroy(acro_index_mapping *m)
{
    return guarded([&] {
        if (m == nullptr) return;
        delete m->m;
        delete m;
    });
}

int *acro_index_mapping_data(acro_index_mapping *m)
{
    return m ? m->m->GetMap().GetData() : nullptr;
}

int acro_index_mapping_compute_inverse(acro_index_mapping *m)
{
    return guarded([&] {
        require(m != nullptr, "null handle");
        m->m->ComputeInverse();
    });
}

int *acro_index_mapping_inverse_data(acro_index_mapping *m)
{
    return (m && m->m->IsInverseComputed()) ? m->m->GetInvMap().GetData() : nullptr;
}

int *acro_index_mapping_inverse_offsets(acro_index_mapping *m)
{
    return (m && m->m->IsInverseComputed()) ? m->m->GetInvMapOffsets().GetData() : nullptr;
}

// ------------------------------------------------------------------------------------------------ engine

int acro_engine_create(const char *exec_type, acro_engine **out)
{
    return guarded([&] {
        require(out != nullptr && exec_type != nullptr, "null argument");
        acro_engine *e = new acro_engine;
        try
        {
            e->te.SetExecutorType(exec_type);
        }
        catch (...)
        {
            delete e;
            throw;
        }
        *out = e;
    });
}

int acro_engine_destroy(acro_engine *e)
{
    return guarded([&] { delete e; });
}

int acro_engine_set_executor_type(acro_engine *e, const char *exec_type)
{
    return guarded([&] {
        require(e != nullptr && exec_type != nullptr, "null argument");
        e->te.SetExecutorType(exec_type);
    });
}

int acro_engine_contract(acro_engine *e, const char *kernel, acro_tensor *out, acro_tensor *const *inputs,
                         int num_inputs)
{
    return guarded([&] {
        require(e != nullptr && kernel != nullptr && out != nullptr, "null argument");
        std::vector<Tensor *> in = unwrap(inputs, num_inputs);
        e->te(std::string(kernel), out->t, in);
        // The call that must not allocate requires this one to have run first on the device; the address of its
        // scratch array is looked up here, where loading code and allocating is allowed.
        if (!e->te.InMultiKernelLaunch()) resolveNoAllocScratch();
    });
}

}  // extern "C"

// ---- the one entry point that allocates nothing ----
// Scratch memory of acro_engine_contract_no_alloc: the kernels of a split contraction keep their per-workgroup partial
// sums (and an arrival counter) in device memory beyond their operands.  The ordinary entry point allocates such a
// buffer per kernel; this array takes its place.  Every device the library runs on holds its own copy, at its own
// address, until the process ends.
#define ACRO_NO_ALLOC_SCRATCH_DOUBLES (ACRO_NO_ALLOC_SCRATCH_BYTES / sizeof(double))
static __device__ __align__(256) double scratch[ACRO_NO_ALLOC_SCRATCH_DOUBLES];

namespace
{
std::mutex scratchLock;
std::map<int, double *> scratchByDevice;

// Device address of `scratch` on the current device; null until resolveNoAllocScratch() has run there.  The array's
// name means nothing as a pointer in host code; only this address is ever handed to kernels and fills.
double *scratchOnCurrentDevice()
{
    int device = 0;
    ACRO_HIP_CHECK(hipGetDevice(&device));
    std::lock_guard<std::mutex> guard(scratchLock);
    auto it = scratchByDevice.find(device);
    return it == scratchByDevice.end() ? nullptr : it->second;
}
}  // namespace

// Looks the address up once per device.  The first look-up on a device may load this library's code object there
// and allocate device memory for it and for the array, so it is done by the ordinary entry point, never by the
// one that promises not to allocate.
static void resolveNoAllocScratch()
{
    int device = 0;
    ACRO_HIP_CHECK(hipGetDevice(&device));
    std::lock_guard<std::mutex> guard(scratchLock);
    if (scratchByDevice.count(device) != 0) return;
    void *address = nullptr;
    ACRO_HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
    require(address != nullptr, "the scratch array has no address on this device");
    scratchByDevice.emplace(device, static_cast<double *>(address));
}

extern "C" {

int acro_engine_contract_no_alloc(acro_engine *e, const char *kernel, acro_tensor *out, acro_tensor *const *inputs,
                                  int num_inputs)
{
    return guarded([&] {
        require(e != nullptr && kernel != nullptr && out != nullptr, "null argument");
        // Inside a multi-kernel launch the call would only be recorded; the launch at its end is an ordinary one.
        require(!e->te.InMultiKernelLaunch(),
                "acro_engine_contract_no_alloc cannot be used between BeginMultiKernelLaunch and EndMultiKernelLaunch");
        std::vector<Tensor *> in = unwrap(inputs, num_inputs);
        double *ptr = scratchOnCurrentDevice();
        require(ptr != nullptr, "acro_engine_contract_no_alloc: nothing has run through acro_engine_contract on this device yet; "
                                "run the same operation once through the ordinary entry point before");
        hip::NoAllocation scope(ptr, ACRO_NO_ALLOC_SCRATCH_DOUBLES);
        e->te(std::string(kernel), out->t, in);
    });
}

int acro_engine_begin_multi_kernel_launch(acro_engine *e)
{
    return guarded([&] {
        require(e != nullptr, "null handle");
        e->te.BeginMultiKernelLaunch();
    });
}

int acro_engine_end_multi_kernel_launch(acro_engine *e)
{
    return guarded([&] {
        require(e != nullptr, "null handle");
        e->te.EndMultiKernelLaunch();
    });
}

int acro_engine_get_implementation(acro_engine *e, const char *kernel, acro_tensor *out, acro_tensor *const *inputs,
                                   int num_inputs, char *buf, size_t buflen, size_t *needed)
{
    return guarded([&] {
        require(e != nullptr && kernel != nullptr && out != nullptr, "null argument");
        std::vector<Tensor *> in = unwrap(inputs, num_inputs);
        copyOut(e->te.GetImplementation(std::string(kernel), out->t, in), buf, buflen, needed);
    });
}

int acro_engine_end_multi_kernel_get_implementation(acro_engine *e, char *buf, size_t buflen, size_t *needed)
{
    return guarded([&] {
        require(e != nullptr, "null handle");
        copyOut(e->te.EndMultiKernelLaunchGetImplementation(), buf, buflen, needed);
    });
}

int acro_engine_get_last_implementation(acro_engine *e, char *buf, size_t buflen, size_t *needed)
{
    return guarded([&] {
        require(e != nullptr, "null handle");
        copyOut(e->te.GetLastImplementation(), buf, buflen, needed);
    });
}

int acro_engine_clear(acro_engine *e)
{
    return guarded([&] {
        require(e != nullptr, "null handle");
        // Clear() also drops the non-contraction ops; re-selecting the policy restores a usable engine.
        std::string type = e->te.GetExecType();
        e->te.SetExecutorType(type);
    });
}

int acro_engine_batch_matrix_inverse(acro_engine *e, acro_tensor *Ainv, acro_tensor *A)
{
    return guarded([&] {
        require(e && Ainv && A, "null handle");
        e->te.BatchMatrixInverse(*Ainv->t, *A->t);
    });
}

int acro_engine_batch_matrix_det(acro_engine *e, acro_tensor *Adet, acro_tensor *A)
{
    return guarded([&] {
        require(e && Adet && A, "null handle");
        e->te.BatchMatrixDet(*Adet->t, *A->t);
    });
}

int acro_engine_batch_matrix_inv_det(acro_engine *e, acro_tensor *Ainv, acro_tensor *Adet, acro_tensor *A)
{
    return guarded([&] {
        require(e && Ainv && Adet && A, "null handle");
        e->te.BatchMatrixInvDet(*Ainv->t, *Adet->t, *A->t);
    });
}

int acro_engine_flat_indexed_scatter(acro_engine *e, acro_tensor *Aout, acro_tensor *Ain, acro_index_mapping *M)
{
    return guarded([&] {
        require(e && Aout && Ain && M, "null handle");
        e->te.FlatIndexedScatter(*Aout->t, *Ain->t, *M->m);
    });
}

int acro_engine_flat_indexed_sum_gather(acro_engine *e, acro_tensor *Aout, acro_tensor *Ain, acro_index_mapping *M)
{
    return guarded([&] {
        require(e && Aout && Ain && M, "null handle");
        e->te.FlatIndexedSumGather(*Aout->t, *Ain->t, *M->m);
    });
}

int acro_hip_compile(const char *module_name, const char *source, size_t *code_size)
{
    return guarded([&] {
        require(module_name != nullptr && source != nullptr, "null argument");
        HipKernel kernel(module_name, source);
        if (code_size != nullptr) *code_size = kernel.GetCodeObjectSize();
    });
}

int acro_hip_compile_private_bytes(const char *module_name, const char *source, const char *function, int *bytes)
{
    return guarded([&] {
        require(module_name != nullptr && source != nullptr && function != nullptr && bytes != nullptr, "null argument");
        HipKernel kernel(module_name, source);
        *bytes = kernel.PrivateSegmentBytes(function);
        require(*bytes >= 0, (std::string("the code object holds no kernel called ") + function).c_str());
    });
}

// ------------------------------------------------------------------------------------- IR introspection

int acro_describe_kernels(int num_kernels, const char *const *kernels, const int *ranks, const int *dims, char *buf,
                          size_t buflen, size_t *needed)
{
    return guarded([&] {
        require(num_kernels > 0 && kernels && ranks && dims, "null argument");
        std::vector<std::unique_ptr<TensorKernel>> parsed;
        std::vector<std::unique_ptr<DimensionedKernel>> bound;
        std::vector<std::unique_ptr<Tensor>> tensors;
        std::vector<double> dummy(1);
        std::vector<DimensionedKernel *> list;
        int ti = 0, di = 0;
        std::ostringstream js;
        js << "{\"kernels\":[";
        for (int k = 0; k < num_kernels; ++k)
        {
            parsed.emplace_back(new TensorKernel(kernels[k]));
            TensorKernel &tk = *parsed.back();
            std::vector<Tensor *> ins;
            Tensor *outT = nullptr;
            for (int v = -1; v < tk.GetNumInputVars(); ++v)
            {
                std::vector<int> d(dims + di, dims + di + ranks[ti]);
                di += ranks[ti++];
                // Shapes only: wrap a one-entry dummy buffer so that nothing large is allocated.
                tensors.emplace_back(new Tensor());
                tensors.back()->Init(d, dummy.data());
                if (v < 0)
                    outT = tensors.back().get();
                else
                    ins.push_back(tensors.back().get());
            }
            std::string dimname = tk.GetDimensionedNameString(outT, ins);
            bound.emplace_back(new DimensionedKernel(&tk, outT, ins));
            DimensionedKernel &dk = *bound.back();
            list.push_back(&dk);
            js << (k ? "," : "") << "{\"name\":\"" << tk.GetNameString() << "\",\"dimensioned_name\":\"" << dimname
               << "\",\"dimensioned_name2\":\"" << dk.GetDimensionedNameString() << "\",\"op\":\"" << tk.EqOperator
               << "\",\"all_indices\":" << jsonList(tk.AllIndexNames)
               << ",\"contraction_indices\":" << jsonList(tk.ContractionIndexNames)
               << ",\"num_outer\":" << tk.GetNumOuterIndices() << ",\"loop_dims\":" << jsonList(dk.GetLoopDims())
               << ",\"flat_size\":" << dk.GetFlatIdxSize() << ",\"out_size\":" << dk.GetOutIdxSize()
               << ",\"cont_size\":" << dk.GetContIdxSize();
            std::vector<int> out_req, in_req;
            for (int nl = 0; nl <= dk.GetNumIndices(); ++nl)
            {
                out_req.push_back(dk.GetOutputStorageReqForInnerLoops(nl));
                in_req.push_back(dk.GetInputStorageReqForInnerLoops(nl));
            }
            js << ",\"out_storage_inner\":" << jsonList(out_req) << ",\"in_storage_inner\":" << jsonList(in_req)
               << ",\"vars\":[";
            for (int v = -1; v < tk.GetNumInputVars(); ++v)
            {
                js << (v >= 0 ? "," : "") << "{\"name\":\"" << tk.GetVarName(v) << "\",\"indices\":"
                   << jsonList(tk.GetVar(v).IndexNames) << ",\"loop_nums\":" << jsonList(tk.GetVar(v).LoopNums)
                   << ",\"size\":" << dk.GetVarSize(v) << "}";
            }
            js << "]}";
        }
        DimensionedMultiKernel mk(list);
        std::vector<std::string> unames;
        for (int u = 0; u < mk.GetNumUVars(); ++u)
        {
            auto first = mk.GetFirstKiVariForUVari(u);
            unames.push_back(mk.Kernels[first.first]->GetVarName(first.second));
        }
        js << "],\"multi\":{\"loop_indices\":" << jsonList(mk.LoopIndices)
           << ",\"shared_outer\":" << jsonList(mk.SharedOuterIndexNames)
           << ",\"contraction_indices\":" << jsonList(mk.ContractionIndexNames)
           << ",\"loop_dims\":" << jsonList(mk.GetLoopDims()) << ",\"unique_vars\":" << jsonList(unames)
           << ",\"dimensioned_name\":\"" << mk.GetDimensionedNameString() << "\"}}";
        copyOut(js.str(), buf, buflen, needed);
    });
}

}  // extern "C"
