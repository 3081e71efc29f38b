// Kernel IR: string -> TensorKernel (parse) -> DimensionedKernel (bind shapes) -> DimensionedMultiKernel (group).
// Semantics follow the reference's kernel/TensorKernel.cpp:26-403, kernel/DimensionedKernel.cpp:12-265 and
// kernel/DimensionedMultiKernel.cpp:25-390; the implementation is a cursor-based scanner plus small index-set
// helpers.
#include <limits>
#include <algorithm>
#include <cctype>
#include <set>

#include "DimensionedMultiKernel.hpp"

namespace acro
{

namespace
{

bool contains(const std::vector<std::string> &list, const std::string &s)
{
    return std::find(list.begin(), list.end(), s) != list.end();
}

void appendUnique(std::vector<std::string> &list, const std::string &s)
{
    if (!contains(list, s)) list.push_back(s);
}

int positionOf(const std::vector<std::string> &list, const std::string &s)
{
    auto it = std::find(list.begin(), list.end(), s);
    return it == list.end() ? -1 : static_cast<int>(it - list.begin());
}

// Scanner over the white-space-free kernel text.  peek() past the end yields '\0', which fails every class test.
class Cursor
{
  public:
    explicit Cursor(const std::string &text) : s(text), pos(0) {}
    char peek() const { return pos < s.size() ? s[pos] : '\0'; }
    char next() { return pos < s.size() ? s[pos++] : '\0'; }
    bool done() const { return pos >= s.size(); }

  private:
    const std::string &s;
    size_t pos;
};

bool isUpper(char c) { return c >= 'A' && c <= 'Z'; }
bool isLowerOrDigit(char c) { return (c >= 'a' && c <= 'z') || (c >= '0' && c <= '9'); }
bool isNameChar(char c) { return isUpper(c) || isLowerOrDigit(c); }

// var := NAME ("_" IDX)+
KernelVar scanVar(Cursor &cur)
{
    KernelVar var;
    ACROBATIC_ASSERT(isUpper(cur.peek()), "Kernel variable names must start with an upper case letter.");
    while (isNameChar(cur.peek())) var.Name += cur.next();
    ACROBATIC_ASSERT(cur.peek() == '_', "Kernel variable " + var.Name + " has no indices.");
    while (cur.peek() == '_')
    {
        cur.next();
        ACROBATIC_ASSERT(isLowerOrDigit(cur.peek()), "Empty index name on kernel variable " + var.Name + ".");
        std::string idx;
        while (isLowerOrDigit(cur.peek())) idx += cur.next();
        var.IndexNames.push_back(idx);
    }
    var.LoopNums.assign(var.IndexNames.size(), 0);
    return var;
}

std::string scanEqOperator(Cursor &cur)
{
    std::string op;
    if (cur.peek() == '+' || cur.peek() == '-') op += cur.next();
    ACROBATIC_ASSERT(cur.peek() == '=', "Expected =, += or -= after the output variable.");
    op += cur.next();
    return op;
}

std::vector<int> rowMajorStrides(const std::vector<int> &dims)
{
    // (the interface has them as int, like the reference's: in a loop space of 2^31 points and more the outer strides
    // saturate instead of overflowing; the generator works with 64-bit strides of its own)
    std::vector<int> strides(dims.size(), 1);
    for (int d = static_cast<int>(dims.size()) - 2; d >= 0; --d)
        strides[d] = static_cast<int>(std::min<long>(std::numeric_limits<int>::max(), static_cast<long>(strides[d + 1]) * dims[d + 1]));
    return strides;
}

}  // namespace

// ---------------------------------------------------------------------------------------- TensorKernel

TensorKernel::TensorKernel(const char *kernel) : KernelStr(kernel)
{
    ParseKernel();
}

TensorKernel::TensorKernel(const std::string &kernel) : KernelStr(kernel)
{
    ParseKernel();
}

TensorKernel::TensorKernel(const std::string &kernel, const std::string &function) : KernelStr(kernel), Function(function)
{
    ParseKernel();
    ACROBATIC_ASSERT(Function.empty() || Function == "inv" || Function == "det", "Unknown kernel function:  " + Function);
    if (Function.empty()) return;
    ACROBATIC_ASSERT(InputVars.size() == 1 && EqOperator == "=", "A matrix kernel assigns a function of one operand:  " + KernelStr);
    const std::vector<std::string> &in = InputVars[0].IndexNames, &out = OutputVar.IndexNames;
    ACROBATIC_ASSERT(in.size() >= 2 && in[in.size() - 1] != in[in.size() - 2], "A matrix kernel needs two distinct trailing indices:  " + KernelStr);
    const std::vector<std::string> lead(in.begin(), in.end() - 2);
    for (size_t a = 0; a < in.size(); ++a)
    {
        for (size_t b = a + 1; b < in.size(); ++b)
            ACROBATIC_ASSERT(in[a] != in[b], "A matrix kernel cannot repeat an index:  " + KernelStr);
    }
    if (Function == "inv")
        ACROBATIC_ASSERT(out == in, "The inverse carries the indices of its operand:  " + KernelStr);
    else
        ACROBATIC_ASSERT(out == lead, "The determinant carries the leading indices of its operand:  " + KernelStr);
}

void TensorKernel::ParseKernel()
{
    std::string text;
    for (char c : KernelStr)
    {
        if (!std::isspace(static_cast<unsigned char>(c))) text += c;
    }

    Cursor cur(text);
    OutputVar = scanVar(cur);
    EqOperator = scanEqOperator(cur);
    do
    {
        InputVars.push_back(scanVar(cur));
    } while (!cur.done());

    for (const auto &idx : OutputVar.IndexNames) appendUnique(AllIndexNames, idx);
    for (const auto &var : InputVars)
    {
        for (const auto &idx : var.IndexNames)
        {
            if (!contains(AllIndexNames, idx))
            {
                ContractionIndexNames.push_back(idx);
                AllIndexNames.push_back(idx);
            }
        }
    }
    // An index repeated inside the output variable (e.g. "A_i_i") still is one loop.
    LoopIndices = AllIndexNames;
    SetVarLoopNums();
}

void TensorKernel::SetVarLoopNums()
{
    auto bind = [this](KernelVar &var) {
        var.LoopNums.resize(var.IndexNames.size());
        for (size_t d = 0; d < var.IndexNames.size(); ++d)
        {
            int pos = positionOf(LoopIndices, var.IndexNames[d]);
            // An index list that omits one of this kernel's indices leaves a number one past the end.
            var.LoopNums[d] = pos < 0 ? static_cast<int>(LoopIndices.size()) : pos;
        }
    };
    bind(OutputVar);
    for (auto &var : InputVars) bind(var);
}

void TensorKernel::SetLoopIndices(const std::vector<std::string> &idx_list)
{
    LoopIndices = idx_list;
    SetVarLoopNums();
}

int TensorKernel::GetVarRank(int vari) const
{
    ACROBATIC_ASSERT(vari >= -1 && vari < GetNumInputVars());
    return static_cast<int>(GetVar(vari).IndexNames.size());
}

int TensorKernel::GetLoopNum(const std::string &idx) const
{
    int pos = positionOf(LoopIndices, idx);
    ACROBATIC_ASSERT(pos >= 0, "Loop index (" + idx + ") not found in kernel:\n" + KernelStr + "\n");
    return pos;
}

int TensorKernel::GetVarDimLoopNum(int vari, int dim) const
{
    ACROBATIC_ASSERT(vari >= -1 && vari < GetNumInputVars());
    ACROBATIC_ASSERT(dim >= 0 && dim < GetVarRank(vari));
    return GetVar(vari).LoopNums[dim];
}

int TensorKernel::GetLoopNumVarDim(int loop_num, int vari) const
{
    ACROBATIC_ASSERT(loop_num >= 0 && loop_num < static_cast<int>(LoopIndices.size()));
    ACROBATIC_ASSERT(vari >= -1 && vari < GetNumInputVars());
    return positionOf(GetVar(vari).IndexNames, LoopIndices[loop_num]);
}

bool TensorKernel::IsVarDependentOnLoop(int vari, int loop_num) const
{
    return GetLoopNumVarDim(loop_num, vari) >= 0;
}

bool TensorKernel::IsDependentOnIndex(const std::string &idx) const
{
    return contains(AllIndexNames, idx);
}

bool TensorKernel::IsDependentOnLoop(int loop_num) const
{
    return IsDependentOnIndex(LoopIndices[loop_num]);
}

bool TensorKernel::IsContractionIndex(const std::string &idx) const
{
    return contains(ContractionIndexNames, idx);
}

bool TensorKernel::IsContractionLoop(int loop_num) const
{
    return IsContractionIndex(LoopIndices[loop_num]);
}

bool TensorKernel::IsContractionVar(int vari) const
{
    ACROBATIC_ASSERT(vari >= -1 && vari < GetNumInputVars());
    if (vari < 0) return false;
    for (const auto &idx : InputVars[vari].IndexNames)
    {
        if (IsContractionIndex(idx)) return true;
    }
    return false;
}

int TensorKernel::GetVarLoopDepth(int vari) const
{
    ACROBATIC_ASSERT(vari >= -1 && vari < GetNumInputVars());
    int depth = -1;
    for (int loop = 0; loop < static_cast<int>(LoopIndices.size()); ++loop)
    {
        if (IsVarDependentOnLoop(vari, loop)) depth = loop;
    }
    return depth;
}

int TensorKernel::GetLoopDepth() const
{
    int depth = -1;
    for (int vari = -1; vari < GetNumInputVars(); ++vari) depth = std::max(depth, GetVarLoopDepth(vari));
    return depth;
}

const std::string &TensorKernel::GetVarName(int vari) const
{
    return GetVar(vari).Name;
}

std::string TensorKernel::GetNameString() const
{
    auto spell = [](const KernelVar &var) {
        std::string s = var.Name;
        for (const auto &idx : var.IndexNames) s += "_" + idx;
        return s;
    };
    std::string name = spell(OutputVar);
    name += (EqOperator == "=") ? "eq" : (EqOperator == "+=") ? "pe" : "me";
    if (!Function.empty()) name += "fn" + Function;
    for (const auto &var : InputVars) name += spell(var);
    return name;
}

std::string TensorKernel::GetDimensionedNameString(Tensor *output, std::vector<Tensor *> &inputs)
{
    std::string name = GetNameString() + "_";
    for (int extent : GetLoopIdxSizes(output, inputs)) name += "_" + std::to_string(extent);
    return name;
}

std::vector<int> TensorKernel::GetLoopIdxSizes(Tensor *output, std::vector<Tensor *> &inputs) const
{
    ACROBATIC_ASSERT(output->GetRank() == GetVarRank(-1),
                     "Tensor rank of the output var in the kernel does not match the rank of the actual tensor.\n"
                     "Kernel:  " + KernelStr);
    ACROBATIC_ASSERT(static_cast<int>(inputs.size()) == GetNumInputVars(),
                     "Number of input tensors does not match the kernel:  " + KernelStr);

    const int nloops = static_cast<int>(LoopIndices.size());
    std::vector<int> extent(nloops, 0);  // 0 = not seen yet
    auto absorb = [&](int vari, const Tensor *t) {
        ACROBATIC_ASSERT(t->GetRank() == GetVarRank(vari),
                         "Tensor rank of input var " + std::to_string(vari) +
                             " does not match the rank of the actual tensor.\nKernel:  " + KernelStr);
        for (int d = 0; d < t->GetRank(); ++d)
        {
            int loop = GetVarDimLoopNum(vari, d);
            ACROBATIC_ASSERT(loop >= 0 && loop < nloops);
            ACROBATIC_ASSERT(extent[loop] == 0 || extent[loop] == t->GetDim(d),
                             "Incompatible tensor dimensions for kernel:  " + KernelStr);
            extent[loop] = t->GetDim(d);
        }
    };
    absorb(-1, output);
    for (int vari = 0; vari < GetNumInputVars(); ++vari) absorb(vari, inputs[vari]);
    for (int &e : extent)
    {
        if (e == 0) e = 1;  // a loop index this kernel does not use
    }
    return extent;
}

// ----------------------------------------------------------------------------------- DimensionedKernel

DimensionedKernel::DimensionedKernel(TensorKernel *kernel, Tensor *output, std::vector<Tensor *> &inputs)
{
    KernelStr = kernel->KernelStr;
    Function = kernel->Function;
    OutputVar = kernel->OutputVar;
    EqOperator = kernel->EqOperator;
    InputVars = kernel->InputVars;
    AllIndexNames = kernel->AllIndexNames;
    ContractionIndexNames = kernel->ContractionIndexNames;
    LoopIndices = kernel->LoopIndices;
    LoopDims = kernel->GetLoopIdxSizes(output, inputs);
    RecomputeStrides();
}

void DimensionedKernel::RecomputeStrides()
{
    LoopStrides = rowMajorStrides(LoopDims);
}

void DimensionedKernel::SetLoopIndices(const std::vector<std::string> &idx_list)
{
    std::vector<int> dims(idx_list.size(), 1);
    for (size_t i = 0; i < idx_list.size(); ++i)
    {
        int old_pos = positionOf(LoopIndices, idx_list[i]);
        if (old_pos >= 0) dims[i] = LoopDims[old_pos];
    }
    LoopDims = dims;
    RecomputeStrides();
    TensorKernel::SetLoopIndices(idx_list);
}

std::string DimensionedKernel::GetLoopDimsString() const
{
    std::string s = "__dim";
    for (const auto &idx : AllIndexNames) s += "_" + std::to_string(GetLoopDim(idx));
    return s;
}

int DimensionedKernel::GetFlatIdxSize() const
{
    int n = 1;
    for (int extent : LoopDims) n *= extent;
    return n;
}

int DimensionedKernel::GetOutIdxSize() const
{
    int n = 1;
    for (int loop = 0; loop < static_cast<int>(LoopDims.size()); ++loop)
    {
        if (IsDependentOnLoop(loop) && !IsContractionLoop(loop)) n *= LoopDims[loop];
    }
    return n;
}

int DimensionedKernel::GetContIdxSize() const
{
    int n = 1;
    for (int loop = 0; loop < static_cast<int>(LoopDims.size()); ++loop)
    {
        if (IsContractionLoop(loop)) n *= LoopDims[loop];
    }
    return n;
}

int DimensionedKernel::GetIdxSizeForFirstNumLoops(int num_loops) const
{
    ACROBATIC_ASSERT(num_loops <= static_cast<int>(LoopDims.size()));
    int n = 1;
    for (int loop = 0; loop < num_loops; ++loop) n *= LoopDims[loop];
    return n;
}

int DimensionedKernel::GetLoopsIdxSize(const std::vector<int> &loops) const
{
    int n = 1;
    for (int loop : loops) n *= LoopDims[loop];
    return n;
}

int DimensionedKernel::GetVarDimStride(int vari, int dim) const
{
    int stride = 1;
    for (int d = GetVarRank(vari) - 1; d > dim; --d) stride *= GetVarDimSize(vari, d);
    return stride;
}

int DimensionedKernel::GetVarSize(int vari) const
{
    int n = 1;
    for (int d = 0; d < GetVarRank(vari); ++d) n *= GetVarDimSize(vari, d);
    return n;
}

int DimensionedKernel::GetVarStorageReqForInnerLoops(int vari, int num_loops) const
{
    const int nloops = static_cast<int>(LoopDims.size());
    ACROBATIC_ASSERT(vari >= -1 && vari < GetNumInputVars());
    ACROBATIC_ASSERT(num_loops >= 0 && num_loops <= nloops);
    int entries = 1;
    for (int loop = nloops - num_loops; loop < nloops; ++loop)
    {
        if (IsVarDependentOnLoop(vari, loop)) entries *= LoopDims[loop];
    }
    return entries;
}

int DimensionedKernel::GetInputStorageReqForInnerLoops(int num_loops) const
{
    int entries = 0;
    for (int vari = 0; vari < GetNumInputVars(); ++vari) entries += GetVarStorageReqForInnerLoops(vari, num_loops);
    return entries;
}

int DimensionedKernel::GetOutputStorageReqForInnerLoops(int num_loops) const
{
    return GetVarStorageReqForInnerLoops(-1, num_loops);
}

int DimensionedKernel::GetTotalStorageReqForInnerLoops(int num_loops) const
{
    return GetInputStorageReqForInnerLoops(num_loops) + GetOutputStorageReqForInnerLoops(num_loops);
}

int DimensionedKernel::GetIndexSpaceSizeForInnerLoops(int num_loops) const
{
    const int nloops = static_cast<int>(LoopDims.size());
    int n = 1;
    for (int loop = nloops - num_loops; loop < nloops; ++loop) n *= LoopDims[loop];
    return n;
}

void DimensionedKernel::GetVarIndexOffsetsForInnerLoops(int vari, int num_inner_loops, std::vector<int> &var_off,
                                                        std::vector<int> &loop_off) const
{
    // Enumerate, in the variable's own dimension order, every combination of those of its indices that run in
    // the innermost num_inner_loops loops; report its offset inside the variable and inside the loop space.
    const int first_inner = static_cast<int>(LoopDims.size()) - num_inner_loops;
    const int rank = GetVarRank(vari);
    std::vector<int> inner_dims;
    for (int d = 0; d < rank; ++d)
    {
        if (GetVarDimLoopNum(vari, d) >= first_inner) inner_dims.push_back(d);
    }
    int count = 1;
    for (int d : inner_dims) count *= GetVarDimSize(vari, d);

    var_off.assign(count, 0);
    loop_off.assign(count, 0);
    for (int n = 0; n < count; ++n)
    {
        int rest = n;
        for (int k = static_cast<int>(inner_dims.size()) - 1; k >= 0; --k)
        {
            int d = inner_dims[k];
            int i = rest % GetVarDimSize(vari, d);
            rest /= GetVarDimSize(vari, d);
            var_off[n] += i * GetVarDimStride(vari, d);
            loop_off[n] += i * LoopStrides[GetVarDimLoopNum(vari, d)];
        }
    }
}

// ------------------------------------------------------------------------------ DimensionedMultiKernel

DimensionedMultiKernel::DimensionedMultiKernel(std::vector<DimensionedKernel *> &kernels) : Kernels(kernels)
{
    InitMKLVars();
}

DimensionedMultiKernel::DimensionedMultiKernel(DimensionedKernel *kernel) : Kernels(1, kernel)
{
    InitMKLVars();
}

void DimensionedMultiKernel::InitMKLVars()
{
    ACROBATIC_ASSERT(!Kernels.empty(), "A multi kernel needs at least one kernel.");

    // Union of indices, union of contraction indices, and the unique-variable table keyed by variable name.
    std::vector<std::string> names;
    for (int ki = 0; ki < GetNumKernels(); ++ki)
    {
        DimensionedKernel *k = Kernels[ki];
        for (const auto &idx : k->AllIndexNames) appendUnique(AllIndexNames, idx);
        for (const auto &idx : k->ContractionIndexNames) appendUnique(ContractionIndexNames, idx);
        for (int vari = -1; vari < k->GetNumInputVars(); ++vari)
        {
            int uvari = positionOf(names, k->GetVarName(vari));
            if (uvari < 0)
            {
                uvari = static_cast<int>(names.size());
                names.push_back(k->GetVarName(vari));
                UVariToFirstKiVari.push_back(std::make_pair(ki, vari));
            }
            KiVariToUVari[std::make_pair(ki, vari)] = uvari;
        }
    }

    // Shared outer indices: carried by every kernel and contracted by none.
    std::vector<std::string> shared;
    for (const auto &idx : AllIndexNames)
    {
        bool ok = true;
        for (DimensionedKernel *k : Kernels) ok = ok && k->IsDependentOnIndex(idx) && !k->IsContractionIndex(idx);
        if (ok) shared.push_back(idx);
    }

    // Largest extent first; equal extents in lexicographic order of the index name.
    std::vector<std::string> sorted(shared.begin(), shared.end());
    std::sort(sorted.begin(), sorted.end());
    std::stable_sort(sorted.begin(), sorted.end(), [this](const std::string &a, const std::string &b) {
        return Kernels[0]->GetLoopDim(a) > Kernels[0]->GetLoopDim(b);
    });
    SharedOuterIndexNames = sorted;

    std::vector<std::string> order = SharedOuterIndexNames;
    for (const auto &idx : AllIndexNames) appendUnique(order, idx);
    SetLoopIndices(order);
}

void DimensionedMultiKernel::SetLoopIndices(const std::vector<std::string> &idx_list)
{
    LoopDims.assign(idx_list.size(), 1);
    for (DimensionedKernel *k : Kernels)
    {
        k->SetLoopIndices(idx_list);
        for (size_t loop = 0; loop < idx_list.size(); ++loop)
        {
            LoopDims[loop] = std::max(LoopDims[loop], k->GetLoopDim(static_cast<int>(loop)));
        }
    }
    LoopStrides = rowMajorStrides(LoopDims);
    LoopIndices = idx_list;
}

int DimensionedMultiKernel::GetNumInputVars() const
{
    int n = 0;
    for (DimensionedKernel *k : Kernels) n += k->GetNumInputVars();
    return n;
}

std::string DimensionedMultiKernel::GetDimensionedNameString() const
{
    std::string name;
    for (DimensionedKernel *k : Kernels) name += k->GetDimensionedNameString() + ";";
    return name;
}

int DimensionedMultiKernel::GetIndexLoopNum(const std::string &idx) const
{
    return positionOf(LoopIndices, idx);
}

int DimensionedMultiKernel::GetVarRank(int ki, int vari) const
{
    return Kernels[ki]->GetVarRank(vari);
}

int DimensionedMultiKernel::GetVarDimLoopNum(int ki, int vari, int dim) const
{
    return Kernels[ki]->GetVarDimLoopNum(vari, dim);
}

int DimensionedMultiKernel::GetLoopNumVarDim(int loop_num, int ki, int vari) const
{
    return Kernels[ki]->GetLoopNumVarDim(loop_num, vari);
}

bool DimensionedMultiKernel::IsVarDependentOnLoop(int ki, int vari, int loop_num) const
{
    return Kernels[ki]->IsVarDependentOnLoop(vari, loop_num);
}

bool DimensionedMultiKernel::IsContractionLoop(int loop_num) const
{
    return contains(ContractionIndexNames, LoopIndices[loop_num]);
}

bool DimensionedMultiKernel::IsSharedOuterLoop(int loop_num) const
{
    return contains(SharedOuterIndexNames, LoopIndices[loop_num]);
}

bool DimensionedMultiKernel::IsOutputUVar(int uvari) const
{
    for (int ki = 0; ki < GetNumKernels(); ++ki)
    {
        if (GetUVari(ki, -1) == uvari) return true;
    }
    return false;
}

bool DimensionedMultiKernel::IsInputUVar(int uvari) const
{
    for (int ki = 0; ki < GetNumKernels(); ++ki)
    {
        for (int vari = 0; vari < Kernels[ki]->GetNumInputVars(); ++vari)
        {
            if (GetUVari(ki, vari) == uvari) return true;
        }
    }
    return false;
}

int DimensionedMultiKernel::GetFlatIdxSize() const
{
    int n = 1;
    for (int extent : LoopDims) n *= extent;
    return n;
}

int DimensionedMultiKernel::GetSharedOuterIdxSize() const
{
    int n = 1;
    for (int loop = 0; loop < GetNumIndices(); ++loop)
    {
        if (IsSharedOuterLoop(loop)) n *= LoopDims[loop];
    }
    return n;
}

int DimensionedMultiKernel::GetIdxSizeForFirstNumLoops(int num_loops) const
{
    int n = 1;
    for (int loop = 0; loop < num_loops; ++loop) n *= LoopDims[loop];
    return n;
}

int DimensionedMultiKernel::GetVarDimStride(int ki, int vari, int dim) const
{
    return Kernels[ki]->GetVarDimStride(vari, dim);
}

int DimensionedMultiKernel::GetVarSize(int ki, int vari) const
{
    return Kernels[ki]->GetVarSize(vari);
}

int DimensionedMultiKernel::GetVarSize(int uvari) const
{
    auto first = UVariToFirstKiVari[uvari];
    return GetVarSize(first.first, first.second);
}

int DimensionedMultiKernel::GetVarLoopDepth(int ki, int vari) const
{
    return Kernels[ki]->GetVarLoopDepth(vari);
}

int DimensionedMultiKernel::GetVarStorageReqForInnerLoops(int ki, int vari, int num_loops) const
{
    return Kernels[ki]->GetVarStorageReqForInnerLoops(vari, num_loops);
}

int DimensionedMultiKernel::GetInputStorageReqForInnerLoops(int num_loops) const
{
    int n = 0;
    for (DimensionedKernel *k : Kernels) n += k->GetInputStorageReqForInnerLoops(num_loops);
    return n;
}

int DimensionedMultiKernel::GetOutputStorageReqForInnerLoops(int num_loops) const
{
    int n = 0;
    for (DimensionedKernel *k : Kernels) n += k->GetOutputStorageReqForInnerLoops(num_loops);
    return n;
}

int DimensionedMultiKernel::GetTotalStorageReqForInnerLoops(int num_loops) const
{
    return GetInputStorageReqForInnerLoops(num_loops) + GetOutputStorageReqForInnerLoops(num_loops);
}

int DimensionedMultiKernel::GetIndexSpaceSizeForInnerLoops(int num_loops) const
{
    int n = 1;
    for (int loop = GetNumIndices() - num_loops; loop < GetNumIndices(); ++loop) n *= LoopDims[loop];
    return n;
}

void DimensionedMultiKernel::GetVarIndexOffsetsForInnerLoops(int ki, int vari, int num_inner_loops,
                                                             std::vector<int> &var_off,
                                                             std::vector<int> &loop_off) const
{
    Kernels[ki]->GetVarIndexOffsetsForInnerLoops(vari, num_inner_loops, var_off, loop_off);
}

}  // namespace acro
