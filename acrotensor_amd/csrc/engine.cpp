// TensorEngine (kernel caches, multi-kernel capture, non-contraction front-ends) and the KernelExecutor base
// class with its policy registry.  Call order and asserts follow the reference's kernel/TensorEngine.cpp:70-95,
// 290-336,538-767 and exec/KernelExecutor.cpp:12-131.
#include <algorithm>
#include <map>

#include "TensorEngine.hpp"

namespace acro
{

// -------------------------------------------------------------------------------------- KernelExecutor

KernelExecutor *CreateHipExecutor(DimensionedMultiKernel *multi_kernel);  // hip_executor.cpp

namespace
{
std::map<std::string, KernelExecutor::Creator> &registry()
{
    static std::map<std::string, KernelExecutor::Creator> table = {{"HIP", &CreateHipExecutor}};
    return table;
}
}  // namespace

KernelExecutor::KernelExecutor(DimensionedMultiKernel *multi_kernel)
    : MultiKernel(multi_kernel), FirstKernel(multi_kernel->Kernels.empty() ? nullptr : multi_kernel->Kernels[0])
{
}

KernelExecutor::~KernelExecutor()
{
    for (size_t ki = 0; ki < SubExecutors.size(); ++ki)
    {
        delete SubExecutors[ki];
        delete SubKernels[ki];
    }
}

void KernelExecutor::Register(const std::string &exec_type, Creator creator)
{
    registry()[exec_type] = creator;
}

bool KernelExecutor::IsRegistered(const std::string &exec_type)
{
    return registry().count(exec_type) > 0;
}

KernelExecutor *KernelExecutor::Create(std::string exec_type, DimensionedMultiKernel *multi_kernel)
{
    auto it = registry().find(exec_type);
    ACROBATIC_ASSERT(it != registry().end(), "Executor type does not exist:  " + exec_type);
    return it->second(multi_kernel);
}

void KernelExecutor::MoveTensorsFromGPU(Tensor *output, std::vector<Tensor *> &inputs)
{
    output->MoveFromGPU();
    for (Tensor *t : inputs) t->MoveFromGPU();
}

void KernelExecutor::MoveTensorsToGPU(Tensor *output, std::vector<Tensor *> &inputs)
{
    // MoveToGPU maps on demand and copies only when the host side holds the current data.
    output->MoveToGPU();
    for (Tensor *t : inputs) t->MoveToGPU();
}

void KernelExecutor::MoveTensorsToOutputLocation(Tensor *output, std::vector<Tensor *> &inputs)
{
    if (output->IsOnGPU())
        MoveTensorsToGPU(output, inputs);
    else
        MoveTensorsFromGPU(output, inputs);
}

void KernelExecutor::ExecuteMulti(std::vector<Tensor *> &output, std::vector<std::vector<Tensor *>> &inputs)
{
    const size_t nk = MultiKernel->Kernels.size();
    if (SubExecutors.size() != nk)
    {
        SubKernels.assign(nk, nullptr);
        SubExecutors.assign(nk, nullptr);
        for (size_t ki = 0; ki < nk; ++ki)
        {
            SubKernels[ki] = new DimensionedMultiKernel(MultiKernel->Kernels[ki]);
            SubExecutors[ki] = KernelExecutor::Create(GetExecType(), SubKernels[ki]);
        }
    }
    for (size_t ki = 0; ki < nk; ++ki) SubExecutors[ki]->ExecuteSingle(output[ki], inputs[ki]);
}

// ---------------------------------------------------------------------------------------- TensorEngine

TensorEngine::TensorEngine() : Ops(nullptr), IsMultiKernelLaunch(false), LastExecutor(nullptr) {}

TensorEngine::TensorEngine(const char *bare_exec_type) : TensorEngine()
{
    SetExecutorType(std::string(bare_exec_type));
}

TensorEngine::TensorEngine(const std::string &exec_type) : TensorEngine()
{
    SetExecutorType(exec_type);
}

TensorEngine::~TensorEngine()
{
    Clear();
}

void TensorEngine::SetExecutorType(const char *bare_exec_type)
{
    SetExecutorType(std::string(bare_exec_type));
}

void TensorEngine::SetExecutorType(const std::string &exec_type)
{
    ACROBATIC_ASSERT(exec_type != "CPUInterpreted" || KernelExecutor::IsRegistered(exec_type),
                     "Executor type CPUInterpreted is not part of this library: it only provides the \"HIP\" "
                     "policy and never computes on the host.");
    ACROBATIC_ASSERT(KernelExecutor::IsRegistered(exec_type), "Unknown Executor type:  " + exec_type);
    // No device work happens here: kernels can be generated and compiled without a device, and the first
    // operation that needs one fails with the HIP error if none is usable.

    Clear();
    ExecutorType = exec_type;
    if (ExecutorType == "HIP")
    {
        ComputeLocation = "GPU";
        Ops = new HipGPUOps();
    }
    else
    {
        ComputeLocation = "CPU";  // a registered host policy brings no non-contraction ops with it
    }
}

void TensorEngine::ResetCapture()
{
    MKLKernels.clear();
    MKLOutputT.clear();
    MKLInputT.clear();
    MKLMatrixOps.clear();
}

void TensorEngine::operator()(const std::string &kernel_str, Tensor *output, std::vector<Tensor *> &inputs)
{
    ACROBATIC_ASSERT(!ExecutorType.empty(), "No executor type has been set on this TensorEngine.");
    ACROBATIC_ASSERT(output->IsInitialized(), "Output variable not initilized in:  " + kernel_str);
    for (Tensor *in : inputs)
    {
        ACROBATIC_ASSERT(in->IsInitialized(), "Input variable not initilized in:  " + kernel_str);
    }

    if (!IsMultiKernelLaunch) ResetCapture();
    TensorKernel *kernel = GetAddTensorKernel(kernel_str);
    MKLKernels.push_back(GetAddDimensionedKernel(kernel, output, inputs));
    MKLOutputT.push_back(output);
    MKLInputT.push_back(inputs);

    if (!IsMultiKernelLaunch)
    {
        LastExecutor = GetAddKernelExecutor();
        LastExecutor->ExecuteSingle(output, inputs);
    }
}

void TensorEngine::BeginMultiKernelLaunch()
{
    ACROBATIC_ASSERT(!IsMultiKernelLaunch, "Trying to BeginMultiKernelLaunch twice.");
    IsMultiKernelLaunch = true;
    ResetCapture();
}

void TensorEngine::EndMultiKernelLaunch()
{
    ACROBATIC_ASSERT(IsMultiKernelLaunch, "Found and EndMultiKernelLaunch before a BeginMultiKernelLaunch!");
    IsMultiKernelLaunch = false;
    FinishCapture(nullptr);
}

// Index and variable names for a recorded matrix operation, taken from the first later kernel that reads its
// result, so that the operation becomes one or two kernels of the group ("Jinv_e_k_m_n = J_e_k_m_n" as an inverse,
// "Jdet_e_k = J_e_k_m_n" as a determinant).  False when no later kernel reads a result, or a result is the operand
// itself: the operation then runs on its own.
bool TensorEngine::MatrixOpAsKernels(const RecordedMatrixOp &op, const std::vector<DimensionedKernel *> &kernels,
                                     const std::vector<Tensor *> &outputs, const std::vector<std::vector<Tensor *>> &inputs,
                                     std::vector<DimensionedKernel *> &op_kernels, std::vector<Tensor *> &op_outputs,
                                     std::vector<std::vector<Tensor *>> &op_inputs)
{
    if (op.inverse == op.matrices || op.determinant == op.matrices) return false;
    const int rank = op.matrices->GetRank();
    std::vector<std::string> lead;
    std::string row, col, inverse_name, determinant_name, matrices_name;
    auto reader = [&](Tensor *t, const KernelVar *&found) {
        found = nullptr;
        for (size_t k = op.position; k < kernels.size() && found == nullptr; ++k)
        {
            for (size_t v = 0; v < inputs[k].size() && found == nullptr; ++v)
            {
                if (inputs[k][v] == t) found = &kernels[k]->GetVar(static_cast<int>(v));
            }
        }
    };
    const KernelVar *inv_reader = nullptr, *det_reader = nullptr;
    if (op.inverse != nullptr) reader(op.inverse, inv_reader);
    if (op.determinant != nullptr) reader(op.determinant, det_reader);
    if (inv_reader != nullptr)
    {
        lead.assign(inv_reader->IndexNames.begin(), inv_reader->IndexNames.end() - 2);
        row = inv_reader->IndexNames[rank - 2];
        col = inv_reader->IndexNames[rank - 1];
        inverse_name = inv_reader->Name;
        if (det_reader != nullptr && det_reader->IndexNames == lead) determinant_name = det_reader->Name;
    }
    else if (det_reader != nullptr)
    {
        lead = det_reader->IndexNames;
        determinant_name = det_reader->Name;
    }
    else
    {
        return false;
    }

    // Names in use anywhere in the capture; made-up names must differ from all of them.
    std::vector<std::string> index_names, var_names;
    for (size_t k = 0; k < kernels.size(); ++k)
    {
        for (int v = -1; v < kernels[k]->GetNumInputVars(); ++v)
        {
            const KernelVar &var = kernels[k]->GetVar(v);
            var_names.push_back(var.Name);
            index_names.insert(index_names.end(), var.IndexNames.begin(), var.IndexNames.end());
            Tensor *t = v < 0 ? outputs[k] : inputs[k][v];
            if (t == op.matrices && matrices_name.empty()) matrices_name = var.Name;
        }
    }
    auto fresh = [](const std::string &stem, std::vector<std::string> &taken) {
        std::string name = stem;
        for (int n = 0; std::find(taken.begin(), taken.end(), name) != taken.end(); ++n) name = stem + std::to_string(n);
        taken.push_back(name);
        return name;
    };
    if (row.empty()) row = fresh("mr", index_names);
    if (col.empty()) col = fresh("mc", index_names);
    if (op.inverse != nullptr && inverse_name.empty()) inverse_name = fresh("MatrixInverse", var_names);
    if (op.determinant != nullptr && determinant_name.empty()) determinant_name = fresh("MatrixDeterminant", var_names);
    if (matrices_name.empty()) matrices_name = fresh("MatrixOperand", var_names);
    std::vector<std::string> all = lead;
    all.push_back(row);
    all.push_back(col);
    for (size_t a = 0; a < all.size(); ++a)
    {
        for (size_t b = a + 1; b < all.size(); ++b)
        {
            if (all[a] == all[b]) return false;  // the reader addresses a diagonal: not a plain copy of the result
        }
    }
    if (inverse_name == matrices_name || determinant_name == matrices_name ||
        (op.inverse != nullptr && op.determinant != nullptr && inverse_name == determinant_name))
        return false;

    auto spell = [](const std::string &name, const std::vector<std::string> &idx) {
        std::string s = name;
        for (const auto &i : idx) s += "_" + i;
        return s;
    };
    std::vector<Tensor *> operand(1, op.matrices);
    if (op.inverse != nullptr)
    {
        TensorKernel *kernel = GetAddTensorKernel(spell(inverse_name, all) + " = " + spell(matrices_name, all), "inv");
        op_kernels.push_back(GetAddDimensionedKernel(kernel, op.inverse, operand));
        op_outputs.push_back(op.inverse);
        op_inputs.push_back(operand);
    }
    if (op.determinant != nullptr)
    {
        TensorKernel *kernel = GetAddTensorKernel(spell(determinant_name, lead) + " = " + spell(matrices_name, all), "det");
        op_kernels.push_back(GetAddDimensionedKernel(kernel, op.determinant, operand));
        op_outputs.push_back(op.determinant);
        op_inputs.push_back(operand);
    }
    return true;
}

void TensorEngine::FinishCapture(std::string *implementation)
{
    std::vector<DimensionedKernel *> kernels;
    std::vector<Tensor *> outputs;
    std::vector<std::vector<Tensor *>> inputs;
    kernels.swap(MKLKernels);
    outputs.swap(MKLOutputT);
    inputs.swap(MKLInputT);
    std::vector<RecordedMatrixOp> ops;
    ops.swap(MKLMatrixOps);

    std::vector<GatheredInput> gathered;  // results of recorded scatters that the kernels read through the maps
    auto flush = [&]() {
        if (MKLKernels.empty()) return;
        KernelExecutor *executor = GetAddKernelExecutor();
        executor->SetGatheredInputs(gathered);
        if (implementation != nullptr)
        {
            *implementation += executor->GetImplementation(MKLOutputT, MKLInputT);
        }
        else
        {
            LastExecutor = executor;
            executor->ExecuteMulti(MKLOutputT, MKLInputT);
        }
        ResetCapture();
    };
    // A recorded scatter need not run when its result is transient, nothing else in the capture writes the result
    // or the source, no kernel recorded before it reads the result, and a kernel recorded after it does.
    auto readThroughMap = [&](const RecordedMatrixOp &op) {
        if (!op.scatter_out->IsTransient() || op.scatter_out == op.scatter_in) return false;
        bool read_later = false;
        for (size_t k = 0; k < kernels.size(); ++k)
        {
            if (outputs[k] == op.scatter_out || outputs[k] == op.scatter_in) return false;
            for (Tensor *t : inputs[k])
            {
                if (t != op.scatter_out) continue;
                if (k < op.position) return false;
                read_later = true;
            }
        }
        for (const auto &other : ops)
        {
            if (&other == &op) continue;
            for (Tensor *t : {other.inverse, other.determinant, other.matrices, other.scatter_out, other.scatter_in})
            {
                if (t == op.scatter_out || (t == op.scatter_in && t != other.scatter_in && t != other.matrices)) return false;
            }
        }
        return read_later;
    };
    // A capture that a matrix operation splits into several launches keeps nothing on chip across them: for its
    // duration no tensor counts as transient (a transient result of one launch may be an operand of the next).
    struct KeepEverything
    {
        std::vector<Tensor *> marked;
        void Add(Tensor *t)
        {
            if (t == nullptr || !t->IsTransient()) return;
            t->SetTransient(false);
            marked.push_back(t);
        }
        ~KeepEverything()
        {
            for (Tensor *t : marked) t->SetTransient(true);
        }
    } keep;
    auto keepAll = [&]() {
        for (size_t k = 0; k < kernels.size(); ++k)
        {
            keep.Add(outputs[k]);
            for (Tensor *t : inputs[k]) keep.Add(t);
        }
        for (const auto &op : ops)
        {
            keep.Add(op.inverse);
            keep.Add(op.determinant);
            keep.Add(op.matrices);
            keep.Add(op.scatter_in);
            bool through_map = false;  // a result that is read through its map stays transient: it is never written
            for (const auto &g : gathered) through_map = through_map || g.operand == op.scatter_out;
            if (!through_map) keep.Add(op.scatter_out);
        }
    };
    size_t next_op = 0;
    for (size_t k = 0; k <= kernels.size(); ++k)
    {
        for (; next_op < ops.size() && ops[next_op].position == k; ++next_op)
        {
            const RecordedMatrixOp &op = ops[next_op];
            if (op.sum_gather)
            {
                // never part of a fused launch (its rows cross workgroups): runs on its own, at its place
                keepAll();
                flush();
                if (implementation != nullptr)
                {
                    *implementation += "// sum-gather: runs on its own\n";
                    continue;
                }
                SwitchToComputeLocation(*op.scatter_out);
                MoveToComputeLocation(*op.scatter_in);
                MoveToComputeLocation(*op.map);
                Ops->FlatIndexedSumGather(*op.scatter_out, *op.scatter_in, *op.map);
                continue;
            }
            if (op.scatter_out != nullptr)
            {
                if (readThroughMap(op))
                {
                    gathered.push_back({op.scatter_out, op.scatter_in, op.map});
                    continue;
                }
                keepAll();
                flush();
                if (implementation != nullptr)
                {
                    *implementation += "// scatter whose result is not transient, or not only read by the kernels after it: runs on its own\n";
                    continue;
                }
                SwitchToComputeLocation(*op.scatter_out);
                MoveToComputeLocation(*op.scatter_in);
                MoveToComputeLocation(*op.map);
                Ops->FlatIndexedScatter(*op.scatter_out, *op.scatter_in, *op.map);
                continue;
            }
            if (MatrixOpAsKernels(op, kernels, outputs, inputs, MKLKernels, MKLOutputT, MKLInputT)) continue;
            keepAll();
            flush();
            if (implementation != nullptr)
            {
                *implementation += "// batched matrix operation whose result no later kernel of the capture reads: runs on its own\n";
                continue;
            }
            if (op.inverse != nullptr) SwitchToComputeLocation(*op.inverse);
            if (op.determinant != nullptr) SwitchToComputeLocation(*op.determinant);
            MoveToComputeLocation(*op.matrices);
            if (op.inverse != nullptr && op.determinant != nullptr)
                Ops->BatchMatrixInvDet(*op.inverse, *op.determinant, *op.matrices);
            else if (op.inverse != nullptr)
                Ops->BatchMatrixInverse(*op.inverse, *op.matrices);
            else
                Ops->BatchMatrixDet(*op.determinant, *op.matrices);
        }
        if (k < kernels.size())
        {
            MKLKernels.push_back(kernels[k]);
            MKLOutputT.push_back(outputs[k]);
            MKLInputT.push_back(inputs[k]);
        }
    }
    flush();
}

std::string TensorEngine::GetImplementation(const std::string &kernel_str, Tensor *output,
                                            std::vector<Tensor *> &inputs)
{
    ACROBATIC_ASSERT(!IsMultiKernelLaunch, "GetImplementation not currently supported for multi kernel launch.");
    ResetCapture();
    TensorKernel *kernel = GetAddTensorKernel(kernel_str);
    MKLKernels.push_back(GetAddDimensionedKernel(kernel, output, inputs));
    MKLOutputT.push_back(output);
    MKLInputT.push_back(inputs);
    return GetAddKernelExecutor()->GetImplementation(MKLOutputT, MKLInputT);
}

std::string TensorEngine::EndMultiKernelLaunchGetImplementation()
{
    ACROBATIC_ASSERT(IsMultiKernelLaunch, "Found and EndMultiKernelLaunch before a BeginMultiKernelLaunch!");
    IsMultiKernelLaunch = false;
    std::string implementation;
    FinishCapture(&implementation);
    return implementation;
}

std::string TensorEngine::GetLastImplementation()
{
    return LastExecutor ? LastExecutor->GetImplementation() : std::string();
}

TensorKernel *TensorEngine::GetAddTensorKernel(const std::string &kernel_str)
{
    auto it = KernelMap.find(kernel_str);
    if (it != KernelMap.end()) return it->second;
    TensorKernel *kernel = new TensorKernel(kernel_str);
    KernelMap[kernel_str] = kernel;
    return kernel;
}

TensorKernel *TensorEngine::GetAddTensorKernel(const std::string &kernel_str, const std::string &function)
{
    const std::string key = kernel_str + " #" + function;  // '#' cannot occur in a kernel string
    auto it = KernelMap.find(key);
    if (it != KernelMap.end()) return it->second;
    TensorKernel *kernel = new TensorKernel(kernel_str, function);
    KernelMap[key] = kernel;
    return kernel;
}

DimensionedKernel *TensorEngine::GetAddDimensionedKernel(TensorKernel *kernel, Tensor *output,
                                                         std::vector<Tensor *> &inputs)
{
    // The same ranks and extents as in the previous call with this kernel string: the same dimensioned kernel (they
    // passed the checks below then).
    DimsOfThisCall.clear();
    auto note = [&](const Tensor *t) {
        DimsOfThisCall.push_back(t->GetRank());
        for (int d = 0; d < t->GetRank(); ++d) DimsOfThisCall.push_back(t->GetDim(d));
    };
    note(output);
    for (const Tensor *t : inputs) note(t);
    DimensionedMemo &memo = LastDimensioned[kernel];
    if (memo.kernel != nullptr && memo.dims == DimsOfThisCall) return memo.kernel;
    // Rank and extent checks happen inside GetLoopIdxSizes, before anything is cached.
    std::string key = kernel->GetDimensionedNameString(output, inputs);
    auto it = DimensionedKernelMap.find(key);
    DimensionedKernel *dk = it != DimensionedKernelMap.end() ? it->second : nullptr;
    if (dk == nullptr)
    {
        dk = new DimensionedKernel(kernel, output, inputs);
        DimensionedKernelMap[key] = dk;
    }
    memo.dims = DimsOfThisCall;
    memo.kernel = dk;
    return dk;
}

KernelExecutor *TensorEngine::GetAddKernelExecutor()
{
    if (LastCaptureExecutor != nullptr && LastCapture == MKLKernels) return LastCaptureExecutor;
    std::string key;
    for (DimensionedKernel *k : MKLKernels) key += k->GetDimensionedNameString() + ";";
    auto it = ExecutorMap.find(key);
    KernelExecutor *executor = it != ExecutorMap.end() ? it->second : nullptr;
    if (executor == nullptr)
    {
        DimensionedMultiKernel *mk = new DimensionedMultiKernel(MKLKernels);
        OwnedMultiKernels.push_back(mk);
        executor = KernelExecutor::Create(ExecutorType, mk);
        ExecutorMap[key] = executor;
    }
    LastCapture = MKLKernels;
    LastCaptureExecutor = executor;
    return executor;
}

namespace
{
void checkInverseShapes(Tensor &Ainv, Tensor &A)
{
    const int rank = A.GetRank();
    ACROBATIC_ASSERT(rank >= 2, "Can't BatchMatrixInverse a tensor of rank < 2.");
    ACROBATIC_ASSERT(rank == Ainv.GetRank(), "Can't BatchMatrixInverse with mismatched ranks for Ainv and A.");
    for (int d = 0; d < rank; ++d)
    {
        ACROBATIC_ASSERT(Ainv.GetDim(d) == A.GetDim(d), "Can't BatchMatrixInverse with mismatched dims for Ainv and A.");
    }
    ACROBATIC_ASSERT(A.GetDim(rank - 1) == A.GetDim(rank - 2), "Can't BatchMatrixInverse with mismatched dims for m,n.");
    ACROBATIC_ASSERT(A.GetDim(rank - 1) <= 3, "Can't BatchMatrixInverse with matrix dims > 3.");
}

void checkDetShapes(Tensor &Adet, Tensor &A)
{
    const int rank = A.GetRank();
    ACROBATIC_ASSERT(rank >= 3, "Can't BatchMatrixDet a tensor of rank < 3.");
    ACROBATIC_ASSERT(Adet.GetRank() == rank - 2, "Can't BatchMatrixDet with mismatched ranks for Adet and A.");
    for (int d = 0; d < rank - 2; ++d)
    {
        ACROBATIC_ASSERT(Adet.GetDim(d) == A.GetDim(d), "Can't BatchMatrixDet with mismatched dims for Adet and A.");
    }
    ACROBATIC_ASSERT(A.GetDim(rank - 1) == A.GetDim(rank - 2), "Can't BatchMatrixDet with mismatched dims for m,n in the matrix.");
    ACROBATIC_ASSERT(A.GetDim(rank - 1) <= 3, "Can't BatchMatrixDet with matrix dims > 3.");
}
}  // namespace

void TensorEngine::BatchMatrixInverse(Tensor &Ainv, Tensor &A)
{
    ACROBATIC_ASSERT(Ops != nullptr, "The executor type of this engine provides no non-contraction ops.");
    checkInverseShapes(Ainv, A);
    if (IsMultiKernelLaunch)
    {
        MKLMatrixOps.push_back({MKLKernels.size(), &Ainv, nullptr, &A, nullptr, nullptr, nullptr});
        return;
    }
    SwitchToComputeLocation(Ainv);
    MoveToComputeLocation(A);
    Ops->BatchMatrixInverse(Ainv, A);
}

void TensorEngine::BatchMatrixDet(Tensor &Adet, Tensor &A)
{
    ACROBATIC_ASSERT(Ops != nullptr, "The executor type of this engine provides no non-contraction ops.");
    checkDetShapes(Adet, A);
    if (IsMultiKernelLaunch)
    {
        MKLMatrixOps.push_back({MKLKernels.size(), nullptr, &Adet, &A, nullptr, nullptr, nullptr});
        return;
    }
    SwitchToComputeLocation(Adet);
    MoveToComputeLocation(A);
    Ops->BatchMatrixDet(Adet, A);
}

void TensorEngine::BatchMatrixInvDet(Tensor &Ainv, Tensor &Adet, Tensor &A)
{
    ACROBATIC_ASSERT(Ops != nullptr, "The executor type of this engine provides no non-contraction ops.");
    checkInverseShapes(Ainv, A);
    checkDetShapes(Adet, A);
    if (IsMultiKernelLaunch)
    {
        MKLMatrixOps.push_back({MKLKernels.size(), &Ainv, &Adet, &A, nullptr, nullptr, nullptr});
        return;
    }
    SwitchToComputeLocation(Ainv);
    SwitchToComputeLocation(Adet);
    MoveToComputeLocation(A);
    Ops->BatchMatrixInvDet(Ainv, Adet, A);
}

void TensorEngine::FlatIndexedScatter(Tensor &Aout, Tensor &Ain, IndexMapping &M)
{
    ACROBATIC_ASSERT(Ops != nullptr, "The executor type of this engine provides no non-contraction ops.");
    ACROBATIC_ASSERT(Aout.GetSize() == static_cast<size_t>(M.GetRangeSize()), "IndexMapping RangeSize does not match the output Tensor size.");
    ACROBATIC_ASSERT(Ain.GetSize() == static_cast<size_t>(M.GetDomainSize()), "IndexMapping DomainSize does not match the input Tensor size.");
    if (IsMultiKernelLaunch && ExecutorType == "HIP")
    {
        MKLMatrixOps.push_back({MKLKernels.size(), nullptr, nullptr, nullptr, &Aout, &Ain, &M});
        return;
    }
    SwitchToComputeLocation(Aout);
    MoveToComputeLocation(Ain);
    MoveToComputeLocation(M);
    Ops->FlatIndexedScatter(Aout, Ain, M);
}

void TensorEngine::FlatIndexedSumGather(Tensor &Aout, Tensor &Ain, IndexMapping &M)
{
    ACROBATIC_ASSERT(Ops != nullptr, "The executor type of this engine provides no non-contraction ops.");
    ACROBATIC_ASSERT(Aout.GetSize() == static_cast<size_t>(M.GetDomainSize()), "IndexMapping DomainSize does not match the output Tensor size.");
    ACROBATIC_ASSERT(Ain.GetSize() == static_cast<size_t>(M.GetRangeSize()), "IndexMapping RangeSize does not match the input Tensor size.");
    if (!M.IsInverseComputed()) M.ComputeInverse();
    if (IsMultiKernelLaunch && ExecutorType == "HIP")
    {
        // Like every other operation of a capture it takes effect at End, at its place among the recorded kernels
        // (run at once, it would gather an operand that the kernels recorded before it have not produced yet).
        RecordedMatrixOp op{MKLKernels.size(), nullptr, nullptr, nullptr, &Aout, &Ain, &M};
        op.sum_gather = true;
        MKLMatrixOps.push_back(op);
        return;
    }
    SwitchToComputeLocation(Aout);
    MoveToComputeLocation(Ain);
    MoveToComputeLocation(M);
    Ops->FlatIndexedSumGather(Aout, Ain, M);
}

void TensorEngine::Clear()
{
    for (auto &e : ExecutorMap) delete e.second;
    ExecutorMap.clear();
    for (DimensionedMultiKernel *mk : OwnedMultiKernels) delete mk;
    OwnedMultiKernels.clear();
    for (auto &k : DimensionedKernelMap) delete k.second;
    DimensionedKernelMap.clear();
    for (auto &k : KernelMap) delete k.second;
    KernelMap.clear();
    delete Ops;
    Ops = nullptr;
    LastExecutor = nullptr;
    LastDimensioned.clear();
    LastCapture.clear();
    LastCaptureExecutor = nullptr;
    ResetCapture();
}

void TensorEngine::MoveToComputeLocation(Tensor &T)
{
    if (ComputeLocation == "GPU")
        T.MoveToGPU();
    else
        T.MoveFromGPU();
}

void TensorEngine::SwitchToComputeLocation(Tensor &T)
{
    if (ComputeLocation == "GPU")
        T.SwitchToGPU();
    else
        T.SwitchFromGPU();
}

void TensorEngine::MoveToComputeLocation(IndexMapping &M)
{
    if (ComputeLocation == "GPU")
        M.MoveToGPU();
    else
        M.MoveFromGPU();
}

}  // namespace acro
