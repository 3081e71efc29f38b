// HipExecutor — the "HIP" execution policy: generates, compiles and launches one fused kernel per
// DimensionedMultiKernel.  Takes the place of the reference's CudaExecutor launch glue
// (exec/CudaExecutor.cpp:17-108: constructor JIT, ExecuteSingle / ExecuteMulti pointer packing, GetImplementation).
//
// Differences that matter to callers:
//  * kernels are generated lazily (first execution or GetImplementation) and per "binding variant": which
//    tensors are transient (their stores may be dropped) and whether any two variables overlap in device memory;
//  * a group that cannot be fused safely (no common outer index, a variable used with different shapes, or
//    overlapping variables of which one is written) is executed as one launch per kernel, in stream order;
//  * everything is enqueued on the library's stream and never synchronised here.
#include <map>
#include <memory>

#include "HipRuntime.hpp"
#include "IndexMapping.hpp"
#include "KernelExecutor.hpp"
#include "NonContractionOps.hpp"
#include "SliceTensor.hpp"
#include "hip_codegen.hpp"
#include "hip_kernel.hpp"

namespace acro
{

class HipExecutor : public KernelExecutor
{
  public:
    explicit HipExecutor(DimensionedMultiKernel *multi_kernel) : KernelExecutor(multi_kernel) {}
    ~HipExecutor() override {}

    std::string GetExecType() override { return "HIP"; }

    std::string GetImplementation() override
    {
        if (LastVariant != nullptr) return Describe(*LastVariant);
        HipCodegenOptions options;
        options.transient.assign(MultiKernel->GetNumUVars(), false);
        return Describe(GetVariant(options));
    }

    std::string GetImplementation(std::vector<Tensor *> &outputs, std::vector<std::vector<Tensor *>> &inputs) override
    {
        HipCodegenOptions options;
        bool fallback = false;
        std::vector<GatheredInput> gathered;
        gathered.swap(Gathered);  // this call only
        Bind(outputs, inputs, gathered, options, fallback);
        if (fallback) return "// not fused (overlapping or re-bound variables): one launch per kernel\n";
        return Describe(GetVariant(options));
    }

    void ExecuteSingle(Tensor *output, std::vector<Tensor *> &inputs) override
    {
        std::vector<Tensor *> outs(1, output);
        std::vector<std::vector<Tensor *>> ins(1, inputs);
        Execute(outs, ins);
    }

    void ExecuteMulti(std::vector<Tensor *> &output, std::vector<std::vector<Tensor *>> &inputs) override
    {
        Execute(output, inputs);
    }

  private:
    struct Variant
    {
        HipKernelPlan plan;
        std::unique_ptr<HipKernel> kernel;  // null when the group is not fusable
        double *scratch = nullptr;          // device buffer shared by the plan's launches
        ~Variant()
        {
            try
            {
                hip::Free(scratch);
            }
            catch (...)
            {
            }
        }
    };

    std::string Describe(const Variant &v)
    {
        if (v.plan.fusable) return v.plan.source;
        return "// not fused (" + v.plan.why_not + "): one launch per kernel\n";
    }

    Variant &GetVariant(const HipCodegenOptions &options)
    {
        std::string key = std::string(options.noalias ? "n" : "a") + (options.positional ? "p" : "u");
        for (bool t : options.transient) key += t ? '1' : '0';
        for (int g : options.gathered) key += "g" + std::to_string(g);
        for (const auto &v : options.views)
        {
            key += "|" + std::to_string(v.storage) + "@" + std::to_string(v.offset);
            for (int d : v.root_dims) key += "," + std::to_string(d);
        }
        auto it = Variants.find(key);
        if (it == Variants.end())
        {
            std::unique_ptr<Variant> v(new Variant);
            v->plan = GenerateHipKernel(*MultiKernel, options);
            if (v->plan.fusable)
            {
                v->kernel.reset(new HipKernel(v->plan.module_name, v->plan.source, v->plan.matrix_core_functions,
                                              v->plan.register_relief_macro));
                if (!v->kernel->PrivateMemoryRemains().empty())
                {
                    // A matrix-core kernel that the compiler could only fit with register spills, also with the
                    // schedule's register-relief switch (or the schedule has none): never launched.  The same group
                    // through the schedules that do without the matrix cores.
                    const std::string refused = v->kernel->PrivateMemoryRemains();
                    HipCodegenOptions plain = options;
                    plain.no_matrix_cores = true;
                    v->plan = GenerateHipKernel(*MultiKernel, plain);
                    v->kernel.reset();
                    if (v->plan.fusable)
                    {
                        const size_t firstLine = v->plan.source.find('\n') + 1;
                        v->plan.source.insert(firstLine, "// (matrix-core kernel " + refused + " needed private memory, i.e. register spills, "
                                                         "and was refused: this is the schedule without the matrix cores)\n");
                        v->kernel.reset(new HipKernel(v->plan.module_name, v->plan.source, v->plan.matrix_core_functions,
                                                      v->plan.register_relief_macro));
                        ACROBATIC_ASSERT(v->kernel->PrivateMemoryRemains().empty(), "Internal error: matrix-core kernel in a plan without matrix cores.");
                    }
                }
                else if (v->kernel->ReliefApplied())
                {
                    v->plan.source = v->kernel->GetSource();  // what was compiled: the relief macro defined in front
                }
            }
            it = Variants.emplace(key, std::move(v)).first;
        }
        LastVariant = it->second.get();
        return *LastVariant;
    }

    // Decides how the tensors of this call bind to kernel operands.  Variables are identified by name, as in the
    // reference's exec/CudaExecutor.cpp:83-99; when one name is bound to two different tensors a group falls back
    // to one launch per kernel and a single kernel switches to one operand per occurrence.  Also the aliasing
    // analysis: two different operands that overlap in memory, one of them written, forbid restrict / scalar
    // reads (single kernel) or fusion (group).  Host buffers mirror library-allocated device buffers one to one, so
    // the analysis works before anything is mapped to the device; device buffers that exist are compared as well.
    void Bind(std::vector<Tensor *> &outputs, std::vector<std::vector<Tensor *>> &inputs,
              const std::vector<GatheredInput> &gathered, HipCodegenOptions &options, bool &fallback)
    {
        const int K = MultiKernel->GetNumKernels();
        ACROBATIC_ASSERT(static_cast<int>(outputs.size()) == K && static_cast<int>(inputs.size()) == K,
                         "Number of tensor lists does not match the number of kernels.");
        auto tensorAt = [&](int ki, int vari) { return vari < 0 ? outputs[ki] : inputs[ki][vari]; };
        auto sameStorage = [](const Tensor *a, const Tensor *b) {
            return a == b || (a->GetData() == b->GetData() && a->GetSize() == b->GetSize());
        };

        bool rebound = false;
        for (int ki = 0; ki < K; ++ki)
        {
            for (int vari = -1; vari < MultiKernel->Kernels[ki]->GetNumInputVars(); ++vari)
            {
                auto first = MultiKernel->GetFirstKiVariForUVari(MultiKernel->GetUVari(ki, vari));
                if (!sameStorage(tensorAt(ki, vari), tensorAt(first.first, first.second))) rebound = true;
            }
        }
        options.positional = (K == 1 && rebound);

        std::vector<Tensor *> operand;
        std::vector<bool> written;
        if (options.positional)
        {
            for (int vari = -1; vari < MultiKernel->Kernels[0]->GetNumInputVars(); ++vari)
            {
                operand.push_back(tensorAt(0, vari));
                written.push_back(vari < 0);
            }
        }
        else
        {
            for (int u = 0; u < MultiKernel->GetNumUVars(); ++u)
            {
                auto first = MultiKernel->GetFirstKiVariForUVari(u);
                operand.push_back(tensorAt(first.first, first.second));
                written.push_back(MultiKernel->IsOutputUVar(u));
            }
        }
        // Storage of every operand: slices are followed up to the tensor they are a view of, so that views of one
        // tensor are recognised as such (the generator resolves them exactly).
        const size_t n = operand.size();
        std::vector<const Tensor *> root(n);
        std::vector<size_t> root_offset(n, 0);
        options.views.assign(n, HipOperandView());
        options.transient.assign(n, false);
        for (size_t a = 0; a < n; ++a)
        {
            const Tensor *t = operand[a];
            while (const SliceTensor *sl = dynamic_cast<const SliceTensor *>(t))
            {
                root_offset[a] += sl->GetOffset();
                t = sl->GetParent();
            }
            root[a] = t;
            options.transient[a] = operand[a]->IsTransient();
            size_t first = a;
            for (size_t b = 0; b < a; ++b)
            {
                if (root[b] == root[a])
                {
                    first = b;
                    break;
                }
            }
            options.views[a].storage = static_cast<int>(first);
            options.views[a].offset = static_cast<long>(root_offset[a]);
            options.views[a].root_dims = root[a]->GetDims();
        }
        // Two different storages that overlap in memory (external buffers) are a hazard when one is written.
        bool hazard = false;
        for (size_t a = 0; a < n; ++a)
        {
            for (size_t b = a + 1; b < n; ++b)
            {
                if (root[a] == root[b]) continue;
                const double *pa = root[a]->GetData(), *pb = root[b]->GetData();
                bool overlap = pa < pb + root[b]->GetSize() && pb < pa + root[a]->GetSize();
                // device buffers that callers handed in need not mirror the layout of the host buffers
                const double *da = root[a]->GetDeviceData(), *db = root[b]->GetDeviceData();
                if (da != nullptr && db != nullptr)
                    overlap = overlap || (da < db + root[b]->GetSize() && db < da + root[a]->GetSize());
                if (overlap && (written[a] || written[b])) hazard = true;
            }
        }
        fallback = K > 1 && (hazard || rebound);
        options.noalias = !hazard;
        // Operands that are read through an index map: whole tensors that the group only reads.
        if (!gathered.empty() && !options.positional && !fallback && !hazard)
        {
            options.gathered.assign(n, -1);
            for (size_t g = 0; g < gathered.size(); ++g)
            {
                for (size_t a = 0; a < n; ++a)
                {
                    if (operand[a] != gathered[g].operand) continue;
                    bool alone = !written[a] && root[a] == operand[a];
                    for (size_t b = 0; b < n; ++b) alone = alone && (b == a || root[b] != root[a]);
                    if (alone) options.gathered[a] = static_cast<int>(g);
                }
            }
        }
    }

    // Runs the scatters whose results the kernels of this call do not read through the maps (`applied`: per operand
    // the pair number the generated code reads, or null when it reads none).
    static void MaterialiseGathered(const std::vector<GatheredInput> &gathered, const std::vector<int> *applied)
    {
        for (size_t g = 0; g < gathered.size(); ++g)
        {
            bool through_map = false;
            if (applied != nullptr)
            {
                for (int slot : *applied) through_map = through_map || slot == static_cast<int>(g);
            }
            if (through_map) continue;
            gathered[g].operand->SwitchToGPU();
            gathered[g].source->MoveToGPU();
            gathered[g].map->MoveToGPU();
            HipGPUOps().FlatIndexedScatter(*gathered[g].operand, *gathered[g].source, *gathered[g].map);
        }
    }

    void Execute(std::vector<Tensor *> &outputs, std::vector<std::vector<Tensor *>> &inputs)
    {
        const int K = MultiKernel->GetNumKernels();
        ACROBATIC_ASSERT(static_cast<int>(outputs.size()) == K && static_cast<int>(inputs.size()) == K,
                         "Number of tensor lists does not match the number of kernels.");
        std::vector<GatheredInput> gathered;
        gathered.swap(Gathered);  // this call only
        // a gathered operand is the result of a scatter: nothing to copy to the device for it
        for (const auto &g : gathered) g.operand->SwitchToGPU();
        for (int ki = 0; ki < K; ++ki) MoveTensorsToGPU(outputs[ki], inputs[ki]);

        // The same tensors in the same places as in the previous call, with the same buffers and marks: the same
        // binding, and the variant it led to (the usual case inside a solver's loop; the analysis below costs several
        // microseconds of host time for a group of kernels, more than a small batch takes on the device).
        ThisCall.clear();
        auto note = [&](const Tensor *t) {
            Seen s;
            s.tensor = t;
            s.host = t->GetData();
            s.device = t->GetDeviceData();
            s.size = static_cast<size_t>(t->GetSize());
            s.transient = t->IsTransient();
            // what Bind derives from a slice's parents: the tensor it is a view of, where, and that tensor's shape
            const Tensor *root = t;
            s.offset = 0;
            while (const SliceTensor *sl = dynamic_cast<const SliceTensor *>(root))
            {
                s.offset += sl->GetOffset();
                root = sl->GetParent();
            }
            s.root = root;
            s.root_device = root->GetDeviceData();
            s.root_shape = 1469598103934665603ull;
            for (int d = 0; d < root->GetRank(); ++d) s.root_shape = (s.root_shape ^ static_cast<unsigned>(root->GetDim(d))) * 1099511628211ull;
            ThisCall.push_back(s);
        };
        for (int ki = 0; ki < K; ++ki)
        {
            note(outputs[ki]);
            for (const Tensor *t : inputs[ki]) note(t);
        }
        const bool repeated = gathered.empty() && LastCallVariant != nullptr && ThisCall == LastCall;
        HipCodegenOptions options;
        if (!repeated)
        {
            LastCallVariant = nullptr;
            bool fallback = false;
            Bind(outputs, inputs, gathered, options, fallback);
            if (fallback)
            {
                MaterialiseGathered(gathered, nullptr);
                KernelExecutor::ExecuteMulti(outputs, inputs);
                return;
            }
        }
        Variant &v = repeated ? *LastCallVariant : GetVariant(options);
        LastVariant = &v;
        if (!v.plan.fusable)
        {
            ACROBATIC_ASSERT(K > 1, "Internal error: a single kernel must always be executable.");
            MaterialiseGathered(gathered, nullptr);
            KernelExecutor::ExecuteMulti(outputs, inputs);
            return;
        }
        if (gathered.empty())
        {
            LastCall.swap(ThisCall);
            LastCallVariant = &v;
        }
        MaterialiseGathered(gathered, v.plan.gathers_applied ? &options.gathered : nullptr);
        std::vector<const int *> gatherMap(gathered.size(), nullptr);
        std::vector<const double *> gatherSource(gathered.size(), nullptr);
        if (v.plan.gathers_applied)
        {
            for (size_t g = 0; g < gathered.size(); ++g)
            {
                gathered[g].source->MoveToGPU();
                gathered[g].map->MoveToGPU();
                gatherMap[g] = gathered[g].map->GetMap().GetDeviceData();
                gatherSource[g] = gathered[g].source->GetDeviceData();
            }
        }
        const size_t nparam = v.plan.param_occurrence.size();
        std::vector<double *> ptr(nparam);
        for (size_t i = 0; i < nparam; ++i)
        {
            const auto &occ = v.plan.param_occurrence[i];
            ptr[i] = (occ.second < 0 ? outputs[occ.first] : inputs[occ.first][occ.second])->GetDeviceData();
            ACROBATIC_ASSERT(ptr[i] != nullptr, "Tensor has no device memory.");
            ptr[i] -= v.plan.param_offset[i];
        }
        double *scratch = nullptr;
        if (v.plan.scratch_doubles > 0 && hip::NoAllocation::Active())
        {
            // The caller's buffer is shared by every operation that runs this way and holds what the last one left
            // there: the part this plan uses starts at zero every time, as a buffer of its own does the first time.
            scratch = hip::NoAllocation::Scratch(v.plan.scratch_doubles);
            hip::FillDouble(scratch, 0.0, v.plan.scratch_doubles);
        }
        else if (v.plan.scratch_doubles > 0)
        {
            if (v.scratch == nullptr)
            {
                v.scratch = static_cast<double *>(hip::Malloc(v.plan.scratch_doubles * sizeof(double)));
                hip::FillDouble(v.scratch, 0.0, v.plan.scratch_doubles);  // on the stream, ahead of the first launch
            }
            scratch = v.scratch;
        }
        for (const auto &z : v.plan.zero_fills)
        {
            hip::FillDouble(ptr[z.param] + z.offset, 0.0, static_cast<size_t>(z.count));
        }
        for (const HipLaunch &launch : v.plan.launches)
        {
            std::vector<void *> args(launch.params.size());
            for (size_t i = 0; i < args.size(); ++i)
            {
                const int code = launch.params[i];
                if (code >= 0)
                    args[i] = static_cast<void *>(&ptr[code]);
                else if (code == -1)
                    args[i] = static_cast<void *>(&scratch);
                else if ((-code - 2) % 2 == 0)
                    args[i] = static_cast<void *>(&gatherMap[(-code - 2) / 2]);
                else
                    args[i] = static_cast<void *>(&gatherSource[(-code - 2) / 2]);
            }
            v.kernel->Launch(launch.function_name, launch.grid, launch.grid_y, launch.block, args.data());
        }
    }

    std::map<std::string, std::unique_ptr<Variant>> Variants;
    Variant *LastVariant = nullptr;
    // one entry per tensor of a call, in call order
    struct Seen
    {
        const Tensor *tensor, *root;
        const double *host, *device, *root_device;
        size_t size, offset;
        unsigned long long root_shape;
        bool transient;
        bool operator==(const Seen &o) const
        {
            return tensor == o.tensor && host == o.host && device == o.device && size == o.size && transient == o.transient &&
                   root == o.root && root_device == o.root_device && offset == o.offset && root_shape == o.root_shape;
        }
    };
    std::vector<Seen> ThisCall, LastCall;
    Variant *LastCallVariant = nullptr;
};

KernelExecutor *CreateHipExecutor(DimensionedMultiKernel *multi_kernel)
{
    return new HipExecutor(multi_kernel);
}

}  // namespace acro
