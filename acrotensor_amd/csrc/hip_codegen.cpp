// Generator: DimensionedMultiKernel -> HIP C++ source (see hip_codegen.hpp for the schedule in words).
// The reference's generator (exec/CudaExecutor.cpp:111-702) maps one CUDA thread to one output entry and loops
// over the contraction reading shared memory twice per multiply-add; this one maps a lane to a pencil of outputs,
// keeps operands in registers / SGPRs and batches several elements per workgroup.
#include "hip_codegen.hpp"

#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <map>
#include <numeric>
#include <set>
#include <sstream>

#include "Error.hpp"

namespace acro
{

namespace
{

// One occurrence of a variable in a kernel.
struct VarRef
{
    int uvar = -1;
    std::vector<int> idx;     // loop id of every dimension
    std::vector<int> ext;     // extent of every dimension
    std::vector<long> stride;  // row-major element stride of every dimension
    long size = 1;
    bool repeated = false;    // some index occurs in two dimensions
};

struct Sub
{
    std::string text;
    VarRef out;
    std::vector<VarRef> in;
    char op = '=';            // '=', '+' or '-'
    std::vector<int> outIdx;  // distinct loop ids of the output
    std::vector<int> contr;   // contraction loop ids, first-appearance order
    // schedule
    std::vector<int> lane;    // loop ids enumerated by the work items (last one fastest)
    std::vector<int> tile;    // loop ids kept in registers by one work item
    bool loopMode = false;    // contraction as counted loops instead of unrolled code
    bool fusedWithPrev = false;
    std::vector<char> forwardedIn;  // per input occurrence: served from the registers of an earlier kernel of the chain
    // 0: contraction.  1: the output is the inverse of the operand's trailing matrix, 2: its determinant.
    int matrixOp = 0;
    int matrixN = 0;
    // > 0: the kernel has one output per batch entry; that many adjacent lanes share its contraction and add their
    // partial sums through lane exchanges
    int splitLanes = 0;
    bool forwardedOld = false;  // the old value of a += / -= output is the previous kernel's result, in registers
    bool flatItems = false;     // one work item per output, numbered as the output lies in memory (no register tile)
    int phase = 0;              // barrier-separated phase the kernel runs in
    long laneCount = 1, tileCount = 1, contrCount = 1;
};

// An operand of the group: a unique variable (by name) or, in positional mode, one occurrence.
struct UVarInfo
{
    std::string name;
    std::vector<int> dims;
    long size = 0;
    bool written = false;
    int firstWrite = -1;
    int lastUse = -1;
    bool consistent = true;       // same shape and batch positions in every occurrence
    std::vector<int> batchDims;   // dimensions carrying the batch index
    bool anyRepeated = false;
    // the storage this operand is a view of
    int storage = -1;
    long viewOffset = 0;          // first element inside the storage
    std::vector<int> fixed;       // leading indices of the storage that the view fixes
    bool plainView = true;        // the view is "leading indices fixed, all trailing dimensions kept"
    bool isVirtual = false;       // intermediate of a factorised kernel: lives in LDS only, no kernel parameter
};

// A tensor's memory: what kernel parameters point to, what LDS tiles mirror and what stores are elided for.
struct Storage
{
    std::vector<int> dims;        // extents of the root tensor
    std::vector<long> stride;     // its row-major strides
    std::vector<int> members;     // operands that are views of it
    bool written = false;
    bool transient = true;        // every member is marked transient
    int batchDim = -1;            // root dimension carrying the batch index
    bool elementLocal = true;     // every member carries the batch index exactly once, at batchDim
    bool anyRepeated = false;
    int firstWrite = -1;          // kernel numbers
    // LDS residency of the per-batch-entry tile
    bool wantLds = false;
    bool inLds = false;
    int tileSize = 0;             // doubles per batch entry
    std::vector<int> ldsStride;   // per root dimension (0 for the batch dimension)
    int ldsOffset = 0;            // in doubles, start of the NB tiles
    int liveTo = -1;              // last kernel that reads the tile from LDS
    int phaseFrom = 0, phaseTo = 0;  // lifetime in barrier-separated phases (fused kernels share a phase)
    bool elide = false;           // no store to device memory
    bool staged = false;          // small input without batch index: every workgroup copies it to LDS before it starts
    bool copyOutOnly = false;     // result that no kernel reads back: its tile only serves to write it out in whole lines
};

long product(const std::vector<int> &ids, const std::vector<int> &extent)
{
    long p = 1;
    for (int i : ids) p *= extent[i];
    return p;
}

bool has(const std::vector<int> &v, int x)
{
    return std::find(v.begin(), v.end(), x) != v.end();
}

std::string str(long v)
{
    return std::to_string(v);
}

uint64_t hashString(const std::string &s)
{
    uint64_t h = 1469598103934665603ull;
    for (unsigned char c : s)
    {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

int envInt(const char *name, int otherwise = 0)
{
    const char *v = std::getenv(name);
    return v ? std::atoi(v) : otherwise;
}

class Generator
{
  public:
    // max_virtual_tile: largest partial result (doubles per batch entry) a reordered single kernel may keep in LDS;
    // 0 = evaluate single kernels as written.
    Generator(const DimensionedMultiKernel &mk_, const HipCodegenOptions &opt_, long max_virtual_tile)
        : mk(mk_), opt(opt_), factorise(max_virtual_tile > 0), maxVirtualTile(max_virtual_tile)
    {
    }

    // The factorised form of a kernel was planned but its intermediates did not all stay on chip: the caller
    // generates the kernel again as written.
    bool factorisationAbandoned = false;

    HipKernelPlan Run()
    {
        HipKernelPlan plan;
        BuildModel();
        std::string why;
        if (!CheckFusable(why))
        {
            plan.fusable = false;
            plan.why_not = why;
            return plan;
        }
        plan.fusable = true;
        if (UseReductionSchedule())
        {
            EmitReduction(plan);
            return plan;
        }
        if (UseTransposeSchedule())
        {
            EmitTranspose(plan);
            return plan;
        }
        if (UseOperatorSchedule())
        {
            EmitOperator(plan);
            return plan;
        }
        ChooseTiles();
        PlanFusion();
        ChooseBatching();
        if (NB == 1 && batch >= 0 && opt.noalias)
        {
            // One batch entry per workgroup makes the batch index uniform across the workgroup: operands that
            // depend on it but on no lane index can then be read with scalar loads too.  Plan again under that
            // assumption and keep the result if it still puts one entry in a workgroup.
            batchUniform = true;
            for (auto &s : subs)
            {
                s.fusedWithPrev = false;
                s.forwardedIn.clear();
                s.forwardedOld = false;
                s.loopMode = false;
            }
            const double busyBefore = busyLanes;
            ChooseTiles();
            PlanFusion();
            ChooseBatching();
            // Scalar operands take their indices out of the lanes; a plan that leaves the wavefronts much emptier than
            // before costs more in issue slots than the scalar loads save (T1_e_q_j_k = B_q_i X_e_i_j_k with X scalar
            // has 6 busy lanes instead of 25: p=4 diffusion apply at 44.8 % of the HBM peak against 72.3 %).
            if (NB != 1 || busyLanes < 0.8 * busyBefore)
            {
                batchUniform = false;
                for (auto &s : subs)
                {
                    s.fusedWithPrev = false;
                    s.forwardedIn.clear();
                    s.forwardedOld = false;
                    s.loopMode = false;
                }
                ChooseTiles();
                PlanFusion();
                ChooseBatching();
            }
        }
        if (factorised)
        {
            for (const auto &st : stores)
            {
                // every read of a partial result must be served from registers or from its LDS tile
                if (uvars[st.members[0]].isVirtual && !st.elide) factorisationAbandoned = true;
            }
            if (factorisationAbandoned)
            {
                plan.fusable = false;
                plan.why_not = "intermediates of the factorised kernel do not fit on chip";
                return plan;
            }
        }
        Emit(plan);
        return plan;
    }

  private:
    const DimensionedMultiKernel &mk;
    const HipCodegenOptions &opt;
    const bool factorise;
    const long maxVirtualTile;
    bool factorised = false;

    int nidx = 0;
    std::vector<std::string> idxName;
    std::vector<int> extent;
    std::vector<Sub> subs;
    std::vector<UVarInfo> uvars;
    std::vector<Storage> stores;
    // Per kernel and input occurrence: every entry it reads has been written to the storage's tile by an earlier
    // kernel of the group (so it can be served from LDS); per kernel: the same for the old value of a += output.
    std::vector<std::vector<bool>> readCovered;
    std::vector<bool> oldCovered;
    int batch = -1;
    long E = 1;
    int NB = 1, NT = 128;
    int ldsDoubles = 0;
    bool extentsConsistent = true;
    bool batchUniform = false;  // one batch entry per workgroup: the batch index is a scalar
    double busyLanes = 1.0;     // share of busy lanes in the wavefronts that the chosen batching issues
    bool lightWorkgroups = false;  // the batch was raised because a workgroup would have moved too few bytes
    bool wide = false;          // 64-bit device-memory offsets

    // Literal of a device-memory stride or offset, and the type such offsets are computed in.
    std::string Lit(long v) const { return std::to_string(v) + (wide ? "L" : ""); }
    const char *OffsetType() const { return wide ? "long" : "int"; }

    // ------------------------------------------------------------------------------------------ model
    // Operand numbering: unique variables by name, or one operand per occurrence in positional mode.
    bool Positional() const { return opt.positional && mk.GetNumKernels() == 1; }
    int NumOperands() const { return Positional() ? mk.Kernels[0]->GetNumVars() : mk.GetNumUVars(); }
    int OperandOf(int ki, int vari) const { return Positional() ? vari + 1 : mk.GetUVari(ki, vari); }
    std::pair<int, int> FirstOccurrence(int u) const
    {
        return Positional() ? std::make_pair(0, u - 1) : mk.GetFirstKiVariForUVari(u);
    }

    void BuildModel()
    {
        nidx = static_cast<int>(mk.LoopIndices.size());
        idxName = mk.LoopIndices;
        extent.assign(nidx, 1);
        for (int i = 0; i < nidx; ++i) extent[i] = mk.GetLoopDim(i);

        uvars.resize(NumOperands());
        const int K = mk.GetNumKernels();
        subs.resize(K);
        for (int ki = 0; ki < K; ++ki)
        {
            DimensionedKernel *k = mk.Kernels[ki];
            Sub &s = subs[ki];
            s.text = k->KernelStr;
            s.op = k->EqOperator[0] == '=' ? '=' : k->EqOperator[0];
            auto makeRef = [&](int vari) {
                VarRef r;
                r.uvar = OperandOf(ki, vari);
                const KernelVar &kv = k->GetVar(vari);
                const int rank = static_cast<int>(kv.IndexNames.size());
                r.idx.resize(rank);
                r.ext.resize(rank);
                r.stride.assign(rank, 1);
                for (int d = 0; d < rank; ++d)
                {
                    r.idx[d] = mk.GetIndexLoopNum(kv.IndexNames[d]);
                    r.ext[d] = k->GetLoopDim(kv.IndexNames[d]);
                    if (r.ext[d] != extent[r.idx[d]]) extentsConsistent = false;
                }
                for (int d = rank - 2; d >= 0; --d) r.stride[d] = r.stride[d + 1] * r.ext[d + 1];
                r.size = 1;
                for (int d = 0; d < rank; ++d) r.size *= r.ext[d];
                std::set<int> distinct(r.idx.begin(), r.idx.end());
                r.repeated = static_cast<int>(distinct.size()) != rank;
                return r;
            };
            s.out = makeRef(-1);
            for (int vari = 0; vari < k->GetNumInputVars(); ++vari) s.in.push_back(makeRef(vari));
            for (int id : s.out.idx)
            {
                if (!has(s.outIdx, id)) s.outIdx.push_back(id);
            }
            for (const auto &name : k->ContractionIndexNames) s.contr.push_back(mk.GetIndexLoopNum(name));
            s.contrCount = product(s.contr, extent);
            if (!k->Function.empty())
            {
                s.matrixOp = k->Function == "inv" ? 1 : 2;
                s.matrixN = s.in[0].ext.back();
                ACROBATIC_ASSERT(s.in[0].ext[s.in[0].ext.size() - 2] == s.matrixN && s.matrixN <= 3,
                                 "HIP generator: a matrix kernel needs square matrices of at most 3 x 3.");
            }
        }

        // The batch index: the largest index that every kernel carries and none contracts (they come sorted), but
        // never a row or column index of a matrix kernel, whose matrices stay whole inside one work item.
        for (const auto &name : mk.SharedOuterIndexNames)
        {
            const int id = mk.GetIndexLoopNum(name);
            bool matrixIndex = false;
            for (const auto &s : subs)
            {
                if (s.matrixOp == 0) continue;
                const std::vector<int> &ids = s.in[0].idx;
                matrixIndex = matrixIndex || id == ids[ids.size() - 1] || id == ids[ids.size() - 2];
            }
            if (matrixIndex) continue;
            batch = id;
            E = extent[batch];
            break;
        }

        if (factorise && envInt("ACRO_HIP_FACTORISE") >= 0) FactoriseKernels();

        // Unique-variable facts, in program order (a kernel reads its inputs before it writes its output).
        for (int ki = 0; ki < static_cast<int>(subs.size()); ++ki)
        {
            const Sub &s = subs[ki];
            auto note = [&](const VarRef &r, bool is_write) {
                UVarInfo &u = uvars[r.uvar];
                std::vector<int> bd;
                for (size_t d = 0; d < r.idx.size(); ++d)
                {
                    if (r.idx[d] == batch) bd.push_back(static_cast<int>(d));
                }
                if (u.lastUse < 0 && u.dims.empty())
                {
                    u.dims = r.ext;
                    u.size = r.size;
                    u.batchDims = bd;
                }
                else if (u.dims != r.ext || u.batchDims != bd)
                {
                    u.consistent = false;
                }
                u.anyRepeated = u.anyRepeated || r.repeated;
                u.lastUse = ki;
                if (is_write)
                {
                    if (!u.written) u.firstWrite = ki;
                    u.written = true;
                }

            };
            for (const auto &r : s.in) note(r, false);
            if (s.op != '=') note(s.out, false);
            note(s.out, true);
        }
        for (int u = 0; u < NumOperands(); ++u)
        {
            auto first = FirstOccurrence(u);
            uvars[u].name = mk.Kernels[first.first]->GetVarName(first.second);
        }
        BuildStorages();
        AnalyseCoverage();
        // Element offsets into device memory are 32-bit unless some tensor of the group reaches 2^31 entries
        // (16 GiB of doubles; the device holds 288 GB): then every device-memory offset is computed in 64 bits.
        for (const auto &st : stores)
        {
            long entries = 1;
            for (int d : st.dims) entries *= d;
            if (entries >= (1L << 31) - 1) wide = true;
        }
    }

    // --------------------------------------------------------------------------- contraction ordering
    // A kernel with three or more operands, written as one big sum
    // ("M_e_i_j_k_l_m_n = B_q_i B_q_l B_r_j B_r_m B_s_k B_s_n W_e_q_r_s": 64 terms of 7 factors for each of 729
    // outputs), is evaluated as a chain of smaller contractions when that takes far fewer multiply-adds: a
    // contraction index is summed as soon as every operand carrying it has been multiplied in, and the partial
    // result becomes the operand of the next step.  The partial results are tensors of the generator's own: one
    // tile per batch entry in LDS, never a kernel parameter.  The steps then run through the same machinery as a
    // user-written multi-kernel group.  The order of the steps is the cheapest (in multiply-adds) among those whose
    // every intermediate carries the batch index and fits in LDS; nothing changes unless the gain is large, because
    // one lane already shares partial sums between the outputs of its pencil.
    static constexpr double kFactoriseMinWork = 8192.0;   // multiply-adds per batch entry as written
    static constexpr double kFactoriseMinGain = 4.0;

    struct FactorStep
    {
        std::vector<int> group;   // operand ids multiplied in this step (inputs: 0..n-1, result of step t: n + t)
        std::vector<int> summed;  // loop ids summed in this step
        std::vector<int> result;  // loop ids of the result, in storage order
    };

    double NonBatchVolume(const std::set<int> &ids) const
    {
        double v = 1.0;
        for (int id : ids)
        {
            if (id != batch) v *= extent[id];
        }
        return v;
    }

    void FactoriseSearch(const Sub &orig, std::vector<int> &live, std::vector<std::vector<int>> &idxOf,
                         std::vector<int> &remaining, double cost, std::vector<FactorStep> &steps, double &best,
                         long &bestSlowest, std::vector<FactorStep> &bestSteps, long &visits) const
    {
        if (++visits > 20000) return;
        // Finish here: one kernel over everything that is left.
        {
            std::set<int> all(orig.outIdx.begin(), orig.outIdx.end());
            for (int o : live) all.insert(idxOf[o].begin(), idxOf[o].end());
            const double total = cost + NonBatchVolume(all) * static_cast<double>(live.size());
            // Among equally cheap orders prefer the one whose last kernel introduces the slowest-varying output
            // indices: they become its register tile, and the lanes then follow the fast output dimensions, which
            // keeps the stores of a wavefront contiguous.
            long slowest = 0;
            const int nin = static_cast<int>(orig.in.size());
            for (size_t d = 0; d < orig.out.idx.size(); ++d)
            {
                const int id = orig.out.idx[d];
                bool inIntermediate = false, inInput = false;
                for (int o : live) (o >= nin ? inIntermediate : inInput) |= has(idxOf[o], id);
                if (id != batch && inInput && !inIntermediate) slowest = slowest == 0 ? orig.out.stride[d] : std::min<long>(slowest, orig.out.stride[d]);
            }
            if (total < best * (1.0 - 1e-9) || (total <= best * (1.0 + 1e-9) && slowest > bestSlowest))
            {
                best = total;
                bestSlowest = slowest;
                bestSteps = steps;
            }
        }
        for (size_t ci = 0; ci < remaining.size(); ++ci)
        {
            const int c = remaining[ci];
            std::vector<int> group, rest;
            for (int o : live) (has(idxOf[o], c) ? group : rest).push_back(o);
            if (rest.empty() || group.empty()) continue;  // that is the final kernel
            std::set<int> all;
            for (int o : group) all.insert(idxOf[o].begin(), idxOf[o].end());
            FactorStep st;
            st.group = group;
            for (int id : remaining)
            {
                if (all.count(id) == 0) continue;
                bool outside = false;
                for (int o : rest) outside = outside || has(idxOf[o], id);
                if (!outside) st.summed.push_back(id);
            }
            std::set<int> kept = all;
            for (int id : st.summed) kept.erase(id);
            if (kept.count(batch) == 0 || NonBatchVolume(kept) > static_cast<double>(maxVirtualTile)) continue;
            const double stepCost = cost + NonBatchVolume(all) * static_cast<double>(group.size());
            if (stepCost > best) continue;
            // Storage order of the result: batch index, the output's indices in the output's order, then the
            // contraction indices still open (read by the next step as literal offsets, unit stride innermost).
            st.result.push_back(batch);
            for (int id : orig.outIdx)
            {
                if (id != batch && kept.count(id)) st.result.push_back(id);
            }
            for (int id : orig.contr)
            {
                if (kept.count(id)) st.result.push_back(id);
            }
            std::vector<int> nextLive = rest, nextRemaining;
            nextLive.push_back(static_cast<int>(idxOf.size()));
            for (int id : remaining)
            {
                if (!has(st.summed, id)) nextRemaining.push_back(id);
            }
            idxOf.push_back(st.result);
            steps.push_back(st);
            FactoriseSearch(orig, nextLive, idxOf, nextRemaining, stepCost, steps, best, bestSlowest, bestSteps, visits);
            steps.pop_back();
            idxOf.pop_back();
        }
    }

    // Every kernel of the group that qualifies is replaced by its steps (a kernel of a multi-kernel launch just as
    // a kernel launched alone).
    void FactoriseKernels()
    {
        std::vector<Sub> expanded;
        int counter = 0;
        for (size_t ki = 0; ki < subs.size(); ++ki)
        {
            if (subs.size() == 1 && ProductThenRowSums(static_cast<int>(ki), subs[ki], expanded, counter)) continue;
            if (!FactoriseKernel(static_cast<int>(ki), subs[ki], subs.size() == 1, expanded, counter)) expanded.push_back(subs[ki]);
        }
        subs.swap(expanded);
    }

    // An element matrix applied to an element vector, "A_e_i = B_e_i_j C_e_j", whose rows are not a multiple of four
    // doubles long (27 x 27): with the lanes along the rows, whether one lane or a few per row, a wavefront reads its
    // matrices in pieces of a row, 216 bytes apart (47 - 53 % of the HBM peak).  Evaluated in two steps instead: the
    // products "_F1_e_i_j = B_e_i_j C_e_j" with the lanes along the matrix as it lies in memory, into a tile in LDS,
    // then the sums over j, one lane per row (a row stride that is odd spreads the lanes over the banks).
    bool ProductThenRowSums(int ki, const Sub &orig, std::vector<Sub> &result, int &counter)
    {
        if (envInt("ACRO_HIP_ROW_SUMS") < 0 || batch < 0 || orig.in.size() != 2 || orig.contr.empty() || !opt.noalias) return false;
        if (orig.out.repeated || orig.matrixOp != 0) return false;
        const VarRef *matrix = nullptr, *vec = nullptr;
        for (const auto &r : orig.in)
        {
            if (r.repeated || r.uvar == orig.out.uvar) return false;
            bool all = has(r.idx, batch);
            for (int id : orig.outIdx) all = all && has(r.idx, id);
            for (int id : orig.contr) all = all && has(r.idx, id);
            if (all && matrix == nullptr)
                matrix = &r;
            else
                vec = &r;
        }
        if (matrix == nullptr || vec == nullptr || matrix == vec) return false;
        // the contraction indices are the matrix's fastest dimensions, the vector carries nothing but them and the batch
        const size_t nc = orig.contr.size();
        if (matrix->idx.size() < nc + 2 || matrix->idx[0] != batch) return false;
        for (size_t d = 0; d < nc; ++d)
        {
            if (!has(orig.contr, matrix->idx[matrix->idx.size() - 1 - d])) return false;
        }
        for (int id : vec->idx)
        {
            if (id != batch && !has(orig.contr, id)) return false;
        }
        const long rows = product(orig.outIdx, extent) / extent[batch], row = orig.contrCount;
        if (row % 4 == 0 || row < 9 || rows < 4 || rows * row > 4096 || row > 512) return false;

        DimensionedKernel *kernel = mk.Kernels[ki];
        auto refText = [&](const std::string &name, const std::vector<int> &ids) {
            std::string t = name;
            for (int id : ids) t += "_" + idxName[id];
            return t;
        };
        UVarInfo info;
        info.isVirtual = true;
        info.name = "_F" + str(static_cast<long>(++counter));
        VarRef res;
        res.uvar = static_cast<int>(uvars.size());
        res.idx = matrix->idx;
        res.ext = matrix->ext;
        res.stride = matrix->stride;
        res.size = matrix->size;
        uvars.push_back(info);

        Sub prod;
        prod.op = '=';
        prod.out = res;
        prod.outIdx = res.idx;
        prod.in = orig.in;
        prod.contrCount = 1;
        prod.flatItems = true;
        prod.text = refText(info.name, res.idx) + " =";
        for (size_t v = 0; v < orig.in.size(); ++v) prod.text += " " + refText(kernel->GetVarName(static_cast<int>(v)), orig.in[v].idx);
        result.push_back(prod);

        Sub fin = orig;
        fin.in.assign(1, res);
        fin.text = refText(kernel->GetVarName(-1), orig.out.idx) + " " + (orig.op == '=' ? "=" : std::string(1, orig.op) + "=") + " " +
                   refText(info.name, res.idx) + "   (steps of: " + orig.text + ")";
        result.push_back(fin);
        factorised = true;
        return true;
    }

    // Appends the steps of kernel ki to `result` and returns true, or returns false when the kernel stays as written.
    bool FactoriseKernel(int ki, const Sub &orig, bool alone, std::vector<Sub> &result, int &counter)
    {
        const int nin = static_cast<int>(orig.in.size());
        if (batch < 0 || nin < 3 || orig.contr.empty() || !opt.noalias || orig.out.repeated) return false;
        if (alone && orig.contrCount >= kReductionMinContraction && product(orig.outIdx, extent) <= kReductionMaxOutputs)
            return false;  // the reduction schedule serves it
        for (const auto &r : orig.in)
        {
            if (r.repeated || r.uvar == orig.out.uvar) return false;
        }
        std::vector<int> live;
        std::vector<std::vector<int>> idxOf;
        for (int v = 0; v < nin; ++v)
        {
            live.push_back(v);
            idxOf.push_back(orig.in[v].idx);
        }
        std::vector<int> remaining = orig.contr;
        std::vector<FactorStep> steps, bestSteps;
        double best = 1e300;
        long visits = 0, bestSlowest = -1;
        std::set<int> all(orig.outIdx.begin(), orig.outIdx.end());
        all.insert(orig.contr.begin(), orig.contr.end());
        const double asWritten = NonBatchVolume(all) * static_cast<double>(nin);
        FactoriseSearch(orig, live, idxOf, remaining, 0.0, steps, best, bestSlowest, bestSteps, visits);
        // ACRO_HIP_FACTORISE=2 (tests): reorder whenever any chain is cheaper at all, however small the kernel.
        const bool eager = envInt("ACRO_HIP_FACTORISE") >= 2;
        if (bestSteps.empty()) return false;
        if (!eager && (asWritten < kFactoriseMinWork || best * kFactoriseMinGain > asWritten)) return false;

        DimensionedKernel *kernel = mk.Kernels[ki];
        auto refText = [&](const std::string &name, const std::vector<int> &ids) {
            std::string t = name;
            for (int id : ids) t += "_" + idxName[id];
            return t;
        };
        std::vector<VarRef> refOf(orig.in.begin(), orig.in.end());
        std::vector<std::string> textOf;
        for (int v = 0; v < nin; ++v) textOf.push_back(refText(kernel->GetVarName(v), orig.in[v].idx));
        std::vector<bool> used(nin, false);
        for (size_t t = 0; t < bestSteps.size(); ++t)
        {
            const FactorStep &st = bestSteps[t];
            UVarInfo info;
            info.isVirtual = true;
            info.name = "_F" + str(static_cast<long>(++counter));
            VarRef res;
            res.uvar = static_cast<int>(uvars.size());
            res.idx = st.result;
            for (int id : st.result) res.ext.push_back(extent[id]);
            res.stride.assign(res.idx.size(), 1);
            for (int d = static_cast<int>(res.idx.size()) - 2; d >= 0; --d) res.stride[d] = res.stride[d + 1] * res.ext[d + 1];
            for (int x : res.ext) res.size *= x;
            uvars.push_back(info);

            Sub s;
            s.op = '=';
            s.out = res;
            s.outIdx = st.result;
            s.contr = st.summed;
            s.contrCount = product(s.contr, extent);
            s.text = refText(info.name, st.result) + " =";
            for (int o : st.group)
            {
                s.in.push_back(refOf[o]);
                s.text += " " + textOf[o];
                used[o] = true;
            }
            result.push_back(s);
            refOf.push_back(res);
            textOf.push_back(refText(info.name, st.result));
            used.push_back(false);
        }
        Sub fin = orig;
        fin.in.clear();
        fin.contr.clear();
        fin.text = refText(kernel->GetVarName(-1), orig.out.idx) + " " + (orig.op == '=' ? "=" : std::string(1, orig.op) + "=");
        for (size_t o = 0; o < refOf.size(); ++o)
        {
            if (used[o]) continue;
            fin.in.push_back(refOf[o]);
            fin.text += " " + textOf[o];
        }
        for (int id : orig.contr)
        {
            bool summedEarlier = false;
            for (const auto &st : bestSteps) summedEarlier = summedEarlier || has(st.summed, id);
            if (!summedEarlier) fin.contr.push_back(id);
        }
        fin.contrCount = product(fin.contr, extent);
        fin.text += "   (steps of: " + orig.text + ")";
        result.push_back(fin);
        factorised = true;
        return true;
    }

    void BuildStorages()
    {
        const int U = static_cast<int>(uvars.size());
        int nstore = 0;
        for (int u = 0; u < U; ++u)
        {
            UVarInfo &op = uvars[u];
            if (static_cast<size_t>(u) < opt.views.size() && opt.views[u].storage >= 0)
            {
                op.storage = opt.views[u].storage;
                op.viewOffset = opt.views[u].offset;
            }
            else
            {
                op.storage = -1 - u;  // renumbered below
            }
        }
        // Dense storage numbers in order of first appearance.
        std::map<int, int> renumber;
        for (int u = 0; u < U; ++u)
        {
            auto it = renumber.find(uvars[u].storage);
            if (it == renumber.end()) it = renumber.emplace(uvars[u].storage, nstore++).first;
            uvars[u].storage = it->second;
        }
        stores.assign(nstore, Storage());
        for (int u = 0; u < U; ++u)
        {
            UVarInfo &op = uvars[u];
            Storage &st = stores[op.storage];
            const bool hasView = static_cast<size_t>(u) < opt.views.size() && !opt.views[u].root_dims.empty();
            if (st.dims.empty())
            {
                st.dims = hasView ? opt.views[u].root_dims : op.dims;
                st.stride.assign(st.dims.size(), 1);
                for (int d = static_cast<int>(st.dims.size()) - 2; d >= 0; --d)
                    st.stride[d] = st.stride[d + 1] * st.dims[d + 1];
            }
            st.members.push_back(u);
            st.written = st.written || op.written;
            st.anyRepeated = st.anyRepeated || op.anyRepeated;
            const bool tr = op.isVirtual || (static_cast<size_t>(u) < opt.transient.size() && opt.transient[u]);
            st.transient = st.transient && tr;
            if (op.written && (st.firstWrite < 0 || op.firstWrite < st.firstWrite)) st.firstWrite = op.firstWrite;

            // The view must be "leading indices fixed, trailing dimensions kept" to be resolved exactly.
            const int nfixed = static_cast<int>(st.dims.size()) - static_cast<int>(op.dims.size());
            op.plainView = nfixed >= 0;
            if (op.plainView)
            {
                for (size_t d = 0; d < op.dims.size(); ++d) op.plainView = op.plainView && st.dims[d + nfixed] == op.dims[d];
                long rest = op.viewOffset;
                op.fixed.assign(nfixed, 0);
                for (int d = 0; d < nfixed; ++d)
                {
                    op.fixed[d] = static_cast<int>(rest / st.stride[d]);
                    rest -= op.fixed[d] * st.stride[d];
                    op.plainView = op.plainView && op.fixed[d] < st.dims[d];
                }
                op.plainView = op.plainView && rest == 0;
            }
            if (!op.plainView || !op.consistent || op.batchDims.size() != 1)
            {
                st.elementLocal = false;
            }
            else
            {
                const int bd = op.batchDims[0] + nfixed;
                if (st.batchDim < 0) st.batchDim = bd;
                if (st.batchDim != bd) st.elementLocal = false;
            }
        }
        for (auto &st : stores)
        {
            if (batch < 0 || st.batchDim < 0) st.elementLocal = false;
            if (!st.elementLocal) continue;
            st.tileSize = 1;
            st.ldsStride.assign(st.dims.size(), 0);
            for (int d = static_cast<int>(st.dims.size()) - 1; d >= 0; --d)
            {
                if (d == st.batchDim) continue;
                st.ldsStride[d] = st.tileSize;
                st.tileSize *= st.dims[d];
            }
        }
    }

    // Is the region "storage at fixed leading indices `fixed`" contained in the union of the written regions?
    bool Covered(const Storage &st, const std::vector<int> &fixed, const std::vector<std::vector<int>> &written) const
    {
        for (const auto &w : written)
        {
            if (w.size() <= fixed.size() && std::equal(w.begin(), w.end(), fixed.begin())) return true;
        }
        const int next = static_cast<int>(fixed.size());
        if (next >= static_cast<int>(st.dims.size()) || next == st.batchDim) return false;
        bool finer = false;
        for (const auto &w : written)
        {
            if (w.size() > fixed.size() && std::equal(fixed.begin(), fixed.end(), w.begin())) finer = true;
        }
        if (!finer) return false;
        std::vector<int> sub = fixed;
        sub.push_back(0);
        for (int v = 0; v < st.dims[next]; ++v)
        {
            sub.back() = v;
            if (!Covered(st, sub, written)) return false;
        }
        return true;
    }

    void AnalyseCoverage()
    {
        const int K = static_cast<int>(subs.size());
        std::vector<std::vector<std::vector<int>>> written(stores.size());
        readCovered.assign(K, std::vector<bool>());
        oldCovered.assign(K, false);
        for (int k = 0; k < K; ++k)
        {
            const Sub &s = subs[k];
            readCovered[k].assign(s.in.size(), false);
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                const UVarInfo &op = uvars[s.in[v].uvar];
                const Storage &st = stores[op.storage];
                readCovered[k][v] = st.elementLocal && op.plainView && Covered(st, op.fixed, written[op.storage]);
            }
            const UVarInfo &oo = uvars[s.out.uvar];
            const Storage &so = stores[oo.storage];
            oldCovered[k] = so.elementLocal && oo.plainView && Covered(so, oo.fixed, written[oo.storage]);
            if (so.elementLocal && oo.plainView && !s.out.repeated) written[oo.storage].push_back(oo.fixed);
        }
    }

    bool CheckFusable(std::string &why)
    {
        if (mk.GetNumKernels() == 1) return true;  // a single kernel always has a private batch index
        for (const auto &s : subs)
        {
            if (s.out.repeated && s.op == '=')
            {
                why = "an assigned output repeats an index and needs a zero fill between kernels";
                return false;
            }
        }
        if (batch < 0)
        {
            why = "the kernels share no outer index";
            return false;
        }
        if (!extentsConsistent)
        {
            why = "an index name has different extents in different kernels";
            return false;
        }
        for (const auto &st : stores)
        {
            // Everything that touches a written tensor must address it through the batch index in one fixed
            // position, or one workgroup would depend on another's results.
            if (st.written && !st.elementLocal)
            {
                why = "variable " + uvars[st.members[0]].name +
                      " is written and used with different shapes, element positions or an unresolvable view";
                return false;
            }
        }
        return true;
    }

    // --------------------------------------------------------------------------------------- schedule
    bool IsPureInput(int uvar) const { return !stores[uvars[uvar].storage].written; }

    // Operand can be read with scalar loads: never written here, no aliasing, small, and its address does not
    // depend on the lane (only on tile / contraction indices, which are literals or uniform loop counters).
    bool IsUniform(const Sub &s, const VarRef &r, const std::vector<int> &tile) const
    {
        if (!opt.noalias || !IsPureInput(r.uvar) || GatherSlot(r.uvar) >= 0) return false;
        bool carriesBatch = false;
        for (int id : r.idx)
        {
            if (id == batch)
            {
                if (!batchUniform) return false;
                carriesBatch = true;
                continue;
            }
            if (!has(tile, id) && !has(s.contr, id)) return false;
        }
        // What one workgroup reads must be small enough to live in the scalar cache.
        const long perEntry = carriesBatch ? r.size / extent[batch] : r.size;
        return perEntry <= 4096;
    }

    // Loads per work item as LoadsPerItem counts them, except for streaming inputs (never written by the group,
    // addressed through the batch index) whose lanes are far apart in memory: their loads are counted as the 16-byte
    // instructions they become, each weighing as many times more as it touches more than 16 lines (four times what
    // a coalesced one touches), if that is more than the plain count.  Measured with one lane per 4 x 4 matrix product against one lane per row: 44.6 against 88.7 % of the HBM
    // peak; "A_e_i = B_e_i_j C_e_j" with 8 x 8: 38.1 against 75.8 %.
    double AccessCostPerItem(const Sub &s, const std::vector<int> &tile) const
    {
        std::vector<int> lanes;
        for (int id : s.out.idx)
        {
            if (id != batch && !has(tile, id) && !has(lanes, id)) lanes.push_back(id);
        }
        double cost = 0.0;
        for (const auto &r : s.in)
        {
            if (IsUniform(s, r, tile)) continue;
            std::set<int> seen;
            long n = 1;
            for (int id : r.idx)
            {
                if ((has(tile, id) || has(s.contr, id)) && seen.insert(id).second) n *= extent[id];
            }
            const bool streams = IsPureInput(r.uvar) && has(r.idx, batch);
            if (!streams)
            {
                cost += static_cast<double>(n);
                continue;
            }
            // trailing dimensions that the work item walks through are contiguous: pairs become 16-byte loads
            long chunk = 1;
            for (size_t d = r.idx.size(); d-- > 0;)
            {
                const int id = r.idx[d];
                if (id == batch || has(lanes, id)) break;
                chunk *= r.ext[d];
            }
            const double instructions = static_cast<double>(n) / chunk * ((chunk + 1) / 2);
            cost += std::max(static_cast<double>(n), instructions * LinesPerInstruction(s, r, lanes) / 16.0);
        }
        return cost;
    }

    long LoadsPerItem(const Sub &s, const std::vector<int> &tile) const
    {
        long loads = 0;
        for (const auto &r : s.in)
        {
            if (IsUniform(s, r, tile)) continue;
            std::set<int> seen;
            long n = 1;
            for (int id : r.idx)
            {
                if ((has(tile, id) || has(s.contr, id)) && seen.insert(id).second) n *= extent[id];
            }
            loads += n;
        }
        return loads;
    }

    // Doubles of streaming operands (inputs that carry the batch index) that one wavefront keeps coming back to: an
    // operand whose fastest dimension is not a lane index is read by each lane in pieces, so the lines that one load
    // instruction touches are touched again by the lane's next loads and have to stay in the CU's 32 KB vector cache
    // in between.  ("A_e_i = B_e_i_j C_e_j" with one lane per entry: 64 lanes x 576 bytes.)
    long WaveFootprint(const Sub &s, const std::vector<int> &tile) const
    {
        std::vector<int> lanes;
        for (int id : s.outIdx)
        {
            if (id != batch && !has(tile, id)) lanes.push_back(id);
        }
        const long perEntry = std::max<long>(1, product(lanes, extent));
        const long entriesPerWave = batch < 0 ? 1 : std::max<long>(1, 64 / perEntry);
        long footprint = 0;
        for (const auto &r : s.in)
        {
            if (!IsPureInput(r.uvar) || !has(r.idx, batch) || IsUniform(s, r, tile) || has(lanes, r.idx.back())) continue;
            std::set<int> seen;
            long perItem = 1, laneSpan = 1;
            for (int id : r.idx)
            {
                if (id == batch || !seen.insert(id).second) continue;
                (has(lanes, id) ? laneSpan : perItem) *= extent[id];
            }
            footprint += std::min<long>(64, laneSpan * entriesPerWave) * perItem;
        }
        return footprint;
    }

    // Average number of 128-byte lines that one load (or store) instruction of the first wavefront touches for
    // occurrence r, the 64 work items being numbered as the emitted code numbers them (batch entries slowest, the
    // last lane index fastest).  Four lines is a fully coalesced access; an operand read in pieces of 8 bytes at a
    // stride of 72 touches 36, and the memory pipeline works through them one by one.
    double LinesPerInstruction(const Sub &s, const VarRef &r, const std::vector<int> &lanes) const
    {
        std::vector<int> literal;  // tile and contraction indices of the occurrence
        for (int id : r.idx)
        {
            if (id != batch && !has(lanes, id) && !has(literal, id)) literal.push_back(id);
        }
        const long combos = product(literal, extent), perEntry = std::max<long>(1, product(lanes, extent));
        const long step = std::max<long>(1, combos / 32);  // a sample of the literal offsets is enough
        std::vector<int> value(nidx, 0);
        double total = 0.0;
        long counted = 0;
        for (long c = 0; c < combos; c += step, ++counted)
        {
            long rem = c;
            for (int j = static_cast<int>(literal.size()) - 1; j >= 0; --j)
            {
                value[literal[j]] = static_cast<int>(rem % extent[literal[j]]);
                rem /= extent[literal[j]];
            }
            std::set<long> lines;
            for (long w = 0; w < 64; ++w)
            {
                const long b = w / perEntry;
                if (b > 0 && (batch < 0 || b >= E)) break;
                long rest = w % perEntry;
                for (int j = static_cast<int>(lanes.size()) - 1; j >= 0; --j)
                {
                    value[lanes[j]] = static_cast<int>(rest % extent[lanes[j]]);
                    rest /= extent[lanes[j]];
                }
                if (batch >= 0) value[batch] = static_cast<int>(b);
                long a = 0;
                for (size_t d = 0; d < r.idx.size(); ++d) a += static_cast<long>(value[r.idx[d]]) * r.stride[d];
                lines.insert(a >> 4);
            }
            total += static_cast<double>(lines.size());
        }
        return counted > 0 ? total / static_cast<double>(counted) : 1.0;
    }

    static constexpr long kUnrollBudget = 8192;   // multiply-adds emitted per work item (before hoisting)
    static constexpr long kMaxUnrolledContraction = 512;  // terms of one unrolled sum
    static constexpr long kMaxTile = 32;
    static constexpr long kMaxLiveValues = 160;   // loaded operands + accumulators held by one lane
    static constexpr long kPrefetchDoubles = 48;  // per lane, held in registers from kernel entry to their phase

    void ChooseTiles()
    {
        for (auto &s : subs)
        {
            s.splitLanes = 0;
            std::vector<int> mid;
            for (int id : s.outIdx)
            {
                if (id != batch) mid.push_back(id);
            }
            const long nin = static_cast<long>(s.in.size());
            if (s.matrixOp != 0)
            {
                // One work item per matrix: the inverse keeps its row and column index as the register tile, the
                // determinant contracts them.
                s.loopMode = false;
                s.tile.clear();
                if (s.matrixOp == 1) s.tile.assign(s.out.idx.end() - 2, s.out.idx.end());
            }
            else if (s.contrCount > kMaxUnrolledContraction || s.contrCount * nin > kUnrollBudget)
            {
                s.loopMode = true;
                s.tile.clear();
            }
            else
            {
                std::vector<std::vector<int>> candidates(1);  // the empty tile
                for (size_t a = 0; a < mid.size(); ++a)
                {
                    candidates.push_back({mid[a]});
                    for (size_t b = a + 1; b < mid.size(); ++b) candidates.push_back({mid[a], mid[b]});
                }
                double bestScore = 1e300;
                std::vector<int> best;
                for (const auto &t : candidates)
                {
                    const long tc = product(t, extent);
                    if (tc > kMaxTile || tc * s.contrCount * nin > kUnrollBudget) continue;
                    const long loads = LoadsPerItem(s, t);
                    if (loads + tc > kMaxLiveValues && !t.empty()) continue;
                    // loads per produced output; a small bias keeps the tile short when nothing is gained
                    const double cost = envInt("ACRO_HIP_FOOTPRINT") >= 0 ? AccessCostPerItem(s, t) : static_cast<double>(loads);
                    double score = cost / tc + 1e-3 * t.size() + 1e-6 * tc;
                    // ... unless the wavefront's working set of partly used lines outgrows its share of the vector cache
                    const long footprint = WaveFootprint(s, t);
                    if (footprint > 512 && envInt("ACRO_HIP_FOOTPRINT") >= 0) score *= static_cast<double>(footprint) / 512.0;
                    if (score < bestScore)
                    {
                        bestScore = score;
                        best = t;
                    }
                }
                // A kernel on its own whose batch entries are tiny (at most 32 outputs, every operand streaming):
                // one output per lane.  The lanes of a wavefront then share the few lines of a handful of entries and
                // every access is coalesced, which outweighs the extra loads (batched 4 x 4 matrix products: 88.7 %
                // of the HBM peak against 55.5 % with a row per lane and 44.6 % with a product per lane; 3 x 3:
                // 64.6 / 58.5 / 53.8 %).
                bool streamingOnly = subs.size() == 1 && batch >= 0 && envInt("ACRO_HIP_FOOTPRINT") >= 0;
                // (small operands without the batch index do not count: they stay in the caches)
                const bool smallInvariantToo = envInt("ACRO_HIP_ONE_OUTPUT") > 0;
                for (const auto &r : s.in)
                    streamingOnly = streamingOnly && (has(r.idx, batch) || (smallInvariantToo && r.size <= 1024)) && !r.repeated;
                const long outputs = product(mid, extent), loadsPerOutput = s.contrCount * nin;
                if (streamingOnly && ((outputs <= 32 && loadsPerOutput <= 16) || (outputs <= 64 && loadsPerOutput <= 4))) best.clear();
                ForcedTile(static_cast<int>(&s - subs.data()), mid, best);
                if (s.flatItems) best.clear();
                s.tile = best;
            }
            SetLanes(s);
            // One output per batch entry ("A_e = B_e_i C_e_i", "A_e = B_e_n"): with one lane per entry every lane walks
            // along its own rows, 8 bytes per line and load instruction (55 and 52 % of the HBM peak).  Instead a power
            // of two of adjacent lanes shares the entry: lane c of them takes the terms c, c + lanes, ... of the
            // flattened contraction, so that the lanes of a wavefront read consecutive addresses, and the partial sums
            // are added in a butterfly of lane exchanges (a fixed order: results are reproducible).  The same for a
            // kernel with few outputs per entry and a contraction along the fastest dimension of a streaming operand
            // ("A_e_i = B_e_i_n", "Y_e_i = M_e_i_j X_e_j" with an element matrix of 27 x 27).
            if (subs.size() == 1 && batch >= 0 && s.matrixOp == 0 && !s.out.repeated && envInt("ACRO_HIP_SPLIT_LANES") >= 0 &&
                !s.contr.empty() && (mid.empty() ? s.contrCount >= 8 : (s.contrCount >= 16 && product(mid, extent) <= 64)))
            {
                // the operand that an entry reads most of carries the batch index and the fastest contraction index last
                const VarRef *most = &s.in[0];
                auto perEntry = [&](const VarRef &r) { return has(r.idx, batch) ? r.size / E : r.size; };
                for (const auto &r : s.in)
                {
                    if (perEntry(r) > perEntry(*most)) most = &r;
                }
                const bool streams = has(most->idx, batch) && most->idx.back() == s.contr.back();
                if (streams)
                {
                    // At most a row of 16 lanes: the exchanges inside a row are register moves, not LDS traffic.  With
                    // several outputs per entry a lane should have at least four terms of its own, or the exchanges
                    // outweigh the arithmetic (16 x 16 matrix-vector products with one term per lane: 47 % against
                    // 59 % unsplit).
                    const long atMost = mid.empty() ? s.contrCount : s.contrCount / 4;
                    int lanes = 1;
                    while (lanes * 2 <= 16 && lanes * 2 <= atMost) lanes *= 2;
                    if (lanes >= (mid.empty() ? 2 : 4))
                    {
                        s.tile.clear();
                        SetLanes(s);
                        s.splitLanes = lanes;
                        s.loopMode = true;
                        s.laneCount *= lanes;
                    }
                }
            }
        }
    }

    // Experiment switch ACRO_HIP_FORCE_TILE="8:;3:q,r": kernel 8 of the group gets the empty register tile, kernel 3
    // the tile (q, r), whatever the cost model says.  Names that are not output indices of the kernel are ignored.
    void ForcedTile(int k, const std::vector<int> &mid, std::vector<int> &tile) const
    {
        const char *spec = std::getenv("ACRO_HIP_FORCE_TILE");
        if (spec == nullptr) return;
        std::istringstream all(spec);
        std::string item;
        while (std::getline(all, item, ';'))
        {
            const size_t colon = item.find(':');
            if (colon == std::string::npos || std::atoi(item.substr(0, colon).c_str()) != k) continue;
            if (!std::isdigit(static_cast<unsigned char>(item[0]))) continue;
            tile.clear();
            std::istringstream names(item.substr(colon + 1));
            std::string name;
            while (std::getline(names, name, ','))
            {
                for (int id : mid)
                {
                    if (idxName[id] == name && !has(tile, id)) tile.push_back(id);
                }
            }
        }
    }

    void SetLanes(Sub &s)
    {
        s.lane.clear();
        // Lane order follows the dimension order of the tensor that should see unit-stride lanes: the output
        // when it is stored to device memory, otherwise the largest operand read from device memory.
        const VarRef *order = &s.out;
        const UVarInfo &uo = uvars[s.out.uvar];
        // read again by a later kernel of the group, under this name or as a view of the same storage
        bool readLater = uo.lastUse > uo.firstWrite;
        for (size_t k2 = static_cast<size_t>(&s - subs.data()) + 1; k2 < subs.size() && !readLater; ++k2)
        {
            for (const auto &r : subs[k2].in) readLater = readLater || ViewsOverlap(r.uvar, s.out.uvar);
        }
        const bool out_stays_on_chip = stores[uo.storage].transient && readLater;
        if (out_stays_on_chip)
        {
            const VarRef *big = nullptr;
            for (const auto &r : s.in)
            {
                if (!IsPureInput(r.uvar) || !has(r.idx, batch)) continue;
                if (big == nullptr || r.size > big->size) big = &r;
            }
            if (big != nullptr) order = big;
        }
        auto consider = [&](int id) {
            if (id == batch || has(s.tile, id) || has(s.lane, id) || !has(s.outIdx, id)) return;
            s.lane.push_back(id);
        };
        for (int id : order->idx) consider(id);
        // Output indices that the ordering tensor does not carry go in front (slowest).
        std::vector<int> front;
        for (int id : s.outIdx)
        {
            if (id != batch && !has(s.tile, id) && !has(s.lane, id)) front.push_back(id);
        }
        s.lane.insert(s.lane.begin(), front.begin(), front.end());
        s.laneCount = product(s.lane, extent);
        s.tileCount = product(s.tile, extent);
    }

    // May operand r of a kernel with lane indices `lane` be taken from the registers in which kernel q left its
    // output?  The work item must be the same (same index wherever q's output carries the batch or a lane index) and
    // the entry must be named at generation time (a tile or contraction index of the reader elsewhere).
    bool ForwardableFrom(const Sub &q, const VarRef &r, const std::vector<int> &lane) const
    {
        if (r.uvar != q.out.uvar || r.idx.size() != q.out.idx.size()) return false;
        for (size_t d = 0; d < r.idx.size(); ++d)
        {
            const int pid = q.out.idx[d];
            const bool itemDim = pid == batch || has(lane, pid);
            if (itemDim ? r.idx[d] != pid : (r.idx[d] == batch || has(lane, r.idx[d]))) return false;
        }
        return true;
    }

    // Kernel k is about to join the chain that starts at chainStart, with lane indices `lane`: the kernels of a chain
    // run one after the other in the same work item without a barrier, so every operand of k that a kernel of the
    // chain writes must be the work item's own entry, taken from registers.  Marks those operands in `fwd`; false
    // when some operand would need another work item's result.
    bool ChainOperandsFromRegisters(int k, int chainStart, const std::vector<int> &lane, std::vector<char> &fwd) const
    {
        const Sub &s = subs[k];
        fwd.assign(s.in.size(), 0);
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            const VarRef &r = s.in[v];
            for (int q = k - 1; q >= chainStart; --q)
            {
                if (!ViewsOverlap(subs[q].out.uvar, r.uvar)) continue;
                if (!ForwardableFrom(subs[q], r, lane)) return false;
                fwd[v] = 1;
                break;
            }
        }
        return true;
    }

    // A kernel whose work items can be those of the previous kernel and that reads results of that kernel (or of
    // the kernels it is itself applied after) entry by entry is applied in the same registers: a pointwise kernel
    // after a contraction ("U = D T3"), but also a small contraction over the register tile of its producer
    // ("D_e_m_n_k = W_k Jdet_e_k Jinv_e_k_n_j Jinv_e_k_m_j" after the inverse and determinant of J_e_k_m_n: one
    // work item per (e, k) holds the nine entries of Jinv).
    void ForwardAlongChain(int k, int chainStart)
    {
        Sub &s = subs[k];
        const Sub &p = subs[k - 1];
        if (envInt("ACRO_HIP_FORWARD") < 0 || p.loopMode || s.loopMode || p.out.repeated || s.out.repeated) return;
        if (s.matrixOp == 2 && p.matrixOp == 1 && s.in[0].uvar == p.in[0].uvar && s.in[0].idx == p.in[0].idx)
        {
            // the determinant of the matrix that the previous kernel inverted: that kernel has computed it
            s.fusedWithPrev = true;
            s.forwardedIn.assign(1, 0);
            s.lane = p.lane;
            s.laneCount = p.laneCount;
            return;
        }
        for (int id : p.lane)
        {
            if (!has(s.outIdx, id)) return;
        }
        std::vector<int> tile;
        for (int id : s.out.idx)
        {
            if (id != batch && !has(p.lane, id) && !has(tile, id)) tile.push_back(id);
        }
        if (s.matrixOp == 1 && tile != std::vector<int>(s.out.idx.end() - 2, s.out.idx.end())) return;
        if (s.matrixOp == 2 && !tile.empty()) return;
        const long tc = product(tile, extent);
        if (tc > kMaxTile || tc * s.contrCount * static_cast<long>(s.in.size()) > kUnrollBudget) return;
        std::vector<char> fwd;
        if (!ChainOperandsFromRegisters(k, chainStart, p.lane, fwd)) return;
        if (std::find(fwd.begin(), fwd.end(), 1) == fwd.end()) return;
        for (int q = chainStart; q < k; ++q)
        {
            if (ViewsOverlap(subs[q].out.uvar, s.out.uvar)) return;
            for (const auto &r : subs[q].in)
            {
                if (ViewsOverlap(r.uvar, s.out.uvar)) return;  // other work items may still read what this one would overwrite
            }
        }
        s.fusedWithPrev = true;
        s.forwardedIn = fwd;
        s.lane = p.lane;
        s.laneCount = p.laneCount;
        s.tile = tile;
        s.tileCount = tc;
    }

    int ChainStartOf(int k) const
    {
        while (k > 0 && subs[k].fusedWithPrev) --k;
        return k;
    }

    void PlanFusion()
    {
        const int K = static_cast<int>(subs.size());
        for (int k = 1; k < K; ++k)
        {
            Sub &s = subs[k];
            const Sub &p = subs[k - 1];
            const int chainStart = ChainStartOf(k - 1);
            // A pointwise kernel over the previous kernel's outputs takes over its lanes and register tile as they are.
            bool pointwise = s.matrixOp == 0 && p.matrixOp == 0 && s.contr.empty() && !p.loopMode && !p.out.repeated && !s.out.repeated;
            if (pointwise)
            {
                std::set<int> a(s.outIdx.begin(), s.outIdx.end()), b(p.outIdx.begin(), p.outIdx.end());
                bool reads = false;
                for (const auto &r : s.in) reads = reads || (r.uvar == p.out.uvar && r.idx == p.out.idx);
                pointwise = a == b && reads && s.out.uvar != p.out.uvar;
            }
            std::vector<char> fwd;
            if (pointwise && ChainOperandsFromRegisters(k, chainStart, p.lane, fwd))
            {
                bool overwrites = false;  // an earlier kernel of the chain reads or writes what this one writes
                for (int q = chainStart; q < k; ++q)
                {
                    overwrites = overwrites || ViewsOverlap(subs[q].out.uvar, s.out.uvar);
                    for (const auto &r : subs[q].in) overwrites = overwrites || ViewsOverlap(r.uvar, s.out.uvar);
                }
                if (!overwrites)
                {
                    s.fusedWithPrev = true;
                    s.forwardedIn = fwd;
                    s.tile = p.tile;
                    s.lane = p.lane;
                    s.laneCount = p.laneCount;
                    s.tileCount = p.tileCount;
                    s.loopMode = false;
                    continue;
                }
            }
            ForwardAlongChain(k, chainStart);
        }
        // Accumulation chains ("Y = ...", "Y += ...", "Y += ..."): a kernel that adds into exactly what the previous
        // kernel produced, with the same pencil decomposition, takes the old value from that kernel's registers.
        for (int k = 1; k < K; ++k)
        {
            Sub &s = subs[k];
            const Sub &p = subs[k - 1];
            if (s.fusedWithPrev || s.op == '=' || s.loopMode || p.loopMode || s.out.repeated) continue;
            if (s.out.uvar != p.out.uvar || s.out.idx != p.out.idx || s.tile != p.tile || s.lane != p.lane) continue;
            std::vector<char> fwd;
            if (!ChainOperandsFromRegisters(k, ChainStartOf(k - 1), p.lane, fwd)) continue;
            s.fusedWithPrev = true;
            s.forwardedIn = fwd;
            s.forwardedOld = true;
        }
        AssignPhases();
    }

    // Two operands address overlapping memory: same storage and neither view's fixed leading indices exclude the
    // other's.
    bool ViewsOverlap(int ua, int ub) const
    {
        const UVarInfo &a = uvars[ua], &b = uvars[ub];
        if (a.storage != b.storage) return false;
        if (!a.plainView || !b.plainView) return true;
        const size_t n = std::min(a.fixed.size(), b.fixed.size());
        for (size_t d = 0; d < n; ++d)
        {
            if (a.fixed[d] != b.fixed[d]) return false;
        }
        return true;
    }

    bool KernelsIndependent(int ka, int kb) const
    {
        const Sub &a = subs[ka], &b = subs[kb];
        if (ViewsOverlap(a.out.uvar, b.out.uvar)) return false;
        for (const auto &r : b.in)
        {
            if (ViewsOverlap(a.out.uvar, r.uvar)) return false;
        }
        for (const auto &r : a.in)
        {
            if (ViewsOverlap(b.out.uvar, r.uvar)) return false;
        }
        return true;
    }

    // Chains (a kernel with the kernels applied in its registers) that do not depend on each other share a phase:
    // their work items are laid side by side across the workgroup's wavefronts, which shortens the sequence of
    // barrier-separated steps one workgroup walks through.
    void AssignPhases()
    {
        const int K = static_cast<int>(subs.size());
        int phase = 0;
        int phaseStart = 0;  // first kernel of the current phase
        for (int k = 0; k < K; ++k)
        {
            if (k > 0 && !subs[k].fusedWithPrev)
            {
                // k opens a new chain: may the whole chain join the current phase?
                int last = k;
                while (last + 1 < K && subs[last + 1].fusedWithPrev) ++last;
                bool join = envInt("ACRO_HIP_MERGE") >= 0 && !subs[k].loopMode;
                for (int a = phaseStart; a < k && join; ++a)
                {
                    if (subs[a].loopMode) join = false;
                    for (int b = k; b <= last && join; ++b) join = KernelsIndependent(a, b);
                }
                if (!join)
                {
                    ++phase;
                    phaseStart = k;
                }
            }
            subs[k].phase = phase;
        }
    }

    bool FromRegisters(int k, int v) const
    {
        return subs[k].fusedWithPrev && static_cast<size_t>(v) < subs[k].forwardedIn.size() && subs[k].forwardedIn[v] != 0;
    }

    int PhaseOf(int k) const { return subs[k].phase; }

    void ComputeLdsWishes()
    {
        const int K = static_cast<int>(subs.size());
        for (auto &st : stores)
        {
            st.wantLds = false;
            st.inLds = false;
            st.liveTo = -1;
            st.staged = false;
            st.copyOutOnly = false;
        }
        if (batch < 0) return;
        ChooseStagedInputs();
        ChooseCopyOutTile();
        for (size_t si = 0; si < stores.size(); ++si)
        {
            Storage &st = stores[si];
            if (!st.written || !st.elementLocal || st.anyRepeated) continue;
            // Last kernel that could take entries of this storage from an LDS tile.
            for (int k = st.firstWrite + 1; k < K; ++k)
            {
                const Sub &s = subs[k];
                for (size_t v = 0; v < s.in.size(); ++v)
                {
                    if (uvars[s.in[v].uvar].storage != static_cast<int>(si)) continue;
                    if (FromRegisters(k, static_cast<int>(v)) || !readCovered[k][v]) continue;
                    st.liveTo = k;
                }
                if (uvars[s.out.uvar].storage == static_cast<int>(si) && s.op != '=' && !s.forwardedOld && oldCovered[k])
                    st.liveTo = k;
            }
            if (st.liveTo < 0 || st.copyOutOnly) continue;
            st.wantLds = true;
            // Kernels fused into one item loop run without a barrier between them, so LDS lifetimes are counted in
            // phases: a tile read in a phase and a tile written in the same phase must not share storage.
            st.phaseFrom = PhaseOf(st.firstWrite);
            st.phaseTo = PhaseOf(st.liveTo);
        }
    }

    // A kernel on its own whose work items each write a long run of consecutive outputs ("A_e_i = B_i_j X_e_j" with a
    // 27 x 3 operator: one lane per entry, 27 results of 216 bytes each) stores pieces of 16 bytes 216 bytes apart:
    // every store instruction of a wavefront touches 64 lines (36 % of the HBM peak).  Its results go to a tile in
    // LDS instead, and after a barrier the whole workgroup writes the tiles of its batch entries, one contiguous range
    // of the tensor, in whole lines.
    void ChooseCopyOutTile()
    {
        if (subs.size() != 1 || envInt("ACRO_HIP_COPY_OUT_TILE") < 0 || envInt("ACRO_HIP_LDS_COPY_OUT") < 0 || envInt("ACRO_HIP_PERSIST") > 0) return;
        const Sub &s = subs[0];
        if (s.loopMode || s.matrixOp != 0 || s.op != '=' || s.out.repeated || s.splitLanes != 0 || s.tile.empty()) return;
        const UVarInfo &u = uvars[s.out.uvar];
        Storage &st = stores[u.storage];
        if (!st.elementLocal || st.anyRepeated || st.members.size() != 1 || st.batchDim != 0 || !u.fixed.empty() || u.viewOffset != 0 || st.transient) return;
        for (const auto &r : s.in)
        {
            if (uvars[r.uvar].storage == u.storage) return;
        }
        // the run of consecutive outputs of one work item: the trailing output dimensions that are tile indices
        long run = 1;
        for (size_t d = s.out.idx.size(); d-- > 0;)
        {
            if (!has(s.tile, s.out.idx[d])) break;
            run *= s.out.ext[d];
        }
        // and the lanes must not interleave at a finer grain (a lane index in the fastest dimension would)
        if (run < 8 || st.tileSize > 2048) return;
        st.copyOutOnly = true;
        st.wantLds = true;
        st.liveTo = 0;
        st.phaseFrom = st.phaseTo = 0;
    }

    // A small operand that does not depend on the batch entry but whose address depends on the lane
    // ("A_e_i = B_i_j X_e_j" with one lane per i: lane i walks along row i of B, 512 bytes from its neighbour's) cannot
    // be read with scalar loads, and read from device memory every load instruction touches 64 lines, which the
    // memory pipeline works through one by one (measured 3 % of the HBM peak for that kernel with a 64 x 64 B).  Every
    // workgroup copies such an operand into LDS once, with coalesced loads, and its lanes read it there; the stride of
    // the lanes in LDS is made odd so that they fall into different banks.
    static constexpr long kMaxStagedDoubles = 4096;

    void ChooseStagedInputs()
    {
        if (envInt("ACRO_HIP_STAGE") < 0 || envInt("ACRO_HIP_PERSIST") > 0 || !opt.noalias) return;
        const int K = static_cast<int>(subs.size());
        for (size_t si = 0; si < stores.size(); ++si)
        {
            Storage &st = stores[si];
            if (st.written || st.members.size() != 1 || st.anyRepeated) continue;
            const UVarInfo &u = uvars[st.members[0]];
            if (!u.consistent || !u.batchDims.empty() || !u.plainView || !u.fixed.empty() || u.isVirtual) continue;
            if (GatherSlot(st.members[0]) >= 0) continue;
            if (u.size > kMaxStagedDoubles || u.size < 64) continue;
            bool ok = true, farApart = false;
            int first = -1, last = -1, laneDim = -1;
            for (int k = 0; k < K && ok; ++k)
            {
                const Sub &sk = subs[k];
                for (size_t v = 0; v < sk.in.size() && ok; ++v)
                {
                    const VarRef &r = sk.in[v];
                    if (uvars[r.uvar].storage != static_cast<int>(si)) continue;
                    if (sk.loopMode || sk.matrixOp != 0 || IsUniform(sk, r, sk.tile)) ok = false;
                    if (!ok) break;
                    if (first < 0)
                    {
                        first = k;
                        for (size_t d = 0; d < r.idx.size(); ++d)
                        {
                            if (has(sk.lane, r.idx[d])) laneDim = static_cast<int>(d);  // fastest dimension that a lane index addresses
                        }
                    }
                    last = k;
                    farApart = farApart || LinesPerInstruction(sk, r, sk.lane) >= 16.0;
                }
                if (uvars[sk.out.uvar].storage == static_cast<int>(si)) ok = false;
            }
            if (!ok || !farApart || first < 0 || laneDim < 0) continue;
            st.staged = true;
            st.wantLds = true;
            st.liveTo = last;
            st.phaseFrom = 0;
            st.phaseTo = PhaseOf(last);
            // row-major, with the run of the dimensions faster than the lanes' made odd
            long run = 1;
            st.ldsStride.assign(st.dims.size(), 0);
            for (int d = static_cast<int>(st.dims.size()) - 1; d >= 0; --d)
            {
                if (d == laneDim && run % 2 == 0) run += 1;
                st.ldsStride[d] = static_cast<int>(run);
                run *= st.dims[d];
            }
            st.tileSize = static_cast<int>(run);
        }
    }

    // Doubles of LDS that a storage's tiles take in a workgroup of nb batch entries.
    int LdsNeed(const Storage &st, int nb) const { return st.tileSize * (st.staged ? 1 : nb); }

    // First-fit placement of the tiles that are live at the same time; returns doubles needed for nb entries.
    int PlaceLds(int nb)
    {
        std::vector<int> order;
        for (size_t si = 0; si < stores.size(); ++si)
        {
            if (stores[si].wantLds && stores[si].inLds) order.push_back(static_cast<int>(si));
        }
        std::sort(order.begin(), order.end(), [&](int a, int b) {
            if (stores[a].phaseFrom != stores[b].phaseFrom) return stores[a].phaseFrom < stores[b].phaseFrom;
            return a < b;
        });
        int total = 0;
        std::vector<int> placed;
        for (int si : order)
        {
            Storage &u = stores[si];
            const int need = LdsNeed(u, nb);
            int offset = 0;
            bool moved = true;
            while (moved)
            {
                moved = false;
                for (int pj : placed)
                {
                    const Storage &p = stores[pj];
                    const bool timeOverlap = !(p.phaseTo < u.phaseFrom || u.phaseTo < p.phaseFrom);
                    const int pneed = LdsNeed(p, nb);
                    const bool spaceOverlap = !(p.ldsOffset + pneed <= offset || offset + need <= p.ldsOffset);
                    if (timeOverlap && spaceOverlap)
                    {
                        offset = p.ldsOffset + pneed;
                        moved = true;
                    }
                }
            }
            u.ldsOffset = offset;
            placed.push_back(si);
            total = std::max(total, offset + need);
        }
        return total;
    }

    void ChooseBatching()
    {
        ComputeLdsWishes();
        long maxLane = 1;
        for (const auto &s : subs) maxLane = std::max(maxLane, s.laneCount);

        NT = opt.force_nt > 0 ? opt.force_nt : envInt("ACRO_HIP_NT");
        if (NT <= 0)
        {
            NT = maxLane > 128 ? 256 : 128;
            // A streaming group (one phase, nothing kept in LDS) with more work items per batch entry than that runs
            // them in one pass of a larger workgroup instead of a loop of passes (geometric-factor setup, 1 000 items:
            // 475.7 -> 457.0 us with 1 024 lanes).  Groups with barriers measured slower that way (p=7 diffusion
            // apply: 1 283 against 940 us), so they keep 256.
            bool streaming = subs.back().phase == 0;
            for (const auto &st : stores) streaming = streaming && !st.wantLds;
            // Not for outputs shared between lanes, whose items are wavefront-sized pieces of rows anyway (64 x 64
            // matrix-vector products: 59 % of the HBM peak with 1 024 lanes, 71 % with 256).
            for (const auto &s : subs) streaming = streaming && s.splitLanes == 0;
            // Larger workgroups leave fewer registers per lane (128 at 1 024 lanes, 256 at 512): size them by the
            // values a lane holds at once.
            long live = 0;
            for (const auto &s : subs) live = std::max(live, s.loopMode ? 8 : LoadsPerItem(s, s.tile) + s.tileCount);
            const long cap = live <= 48 ? 1024 : (live <= 100 ? 512 : 256);
            if (streaming && maxLane > 256) NT = static_cast<int>(std::min<long>(cap, (maxLane + 63) / 64 * 64));
        }
        NB = opt.force_nb > 0 ? opt.force_nb : envInt("ACRO_HIP_NB");
        if (NB <= 0)
        {
            // As many batch entries as fit in one pass of the widest kernel, rounded down to a power of two.
            long fit = std::max<long>(1, NT / maxLane);
            NB = 1;
            while (NB * 2 <= fit) NB *= 2;
        }
        if (batch < 0) NB = 1;
        NB = static_cast<int>(std::min<long>(NB, E));

        // Lane utilisation at wavefront granularity (a wavefront with a single busy lane costs as much issue time as
        // a full one).  When the default leaves many lanes idle, look for a batch size / workgroup size that packs
        // wavefronts better; only switch for a clear gain, small workgroups overlap memory latency better.
        if (opt.force_nb <= 0 && opt.force_nt <= 0 && envInt("ACRO_HIP_NB") <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0)
        {
            auto utilisation = [&](int nb, int nt) {
                double busy = 0.0, issued = 0.0;
                for (const auto &s : subs)
                {
                    if (s.fusedWithPrev) continue;
                    const long items = static_cast<long>(nb) * s.laneCount;
                    const long passes = (items + nt - 1) / nt;
                    const long tail = items - (passes - 1) * nt;
                    const double weight = static_cast<double>(std::max<long>(1, s.tileCount * s.contrCount));
                    busy += weight * items;
                    issued += weight * 64.0 * ((passes - 1) * (nt / 64) + (tail + 63) / 64);
                }
                return busy / issued;
            };
            // Share of the arithmetic in kernels that need more than one pass of the workgroup over their items.
            auto multiPassShare = [&](int nb, int nt) {
                double all = 0.0, looped = 0.0;
                for (const auto &s : subs)
                {
                    const double work = static_cast<double>(s.laneCount) * std::max<long>(1, s.tileCount * s.contrCount);
                    all += work;
                    if (static_cast<long>(nb) * s.laneCount > nt) looped += work;
                }
                return all > 0.0 ? looped / all : 0.0;
            };
            // Workgroups that declare much LDS leave few wavefronts resident on a compute unit (160 KB of LDS, handed
            // out in 1280-byte granules, 32 wavefronts at most) and so fewer loads in flight to cover the memory
            // latency; the square root follows the measured rates (p=3 diffusion apply in 256 lanes: 77.3 % of the
            // HBM peak with 32 resident wavefronts, 69.8 % with 12 and fuller wavefronts).
            auto occupancy = [&](int nb, int nt) {
                long bytes = static_cast<long>(PlaceLds(nb)) * 8;
                bytes = std::max<long>(1280, (bytes + 1279) / 1280 * 1280);
                const long groups = std::min<long>(160 * 1024 / bytes, 32 / (nt / 64));
                // wavefronts of a workgroup that have items at all, averaged over the arithmetic
                double all = 0.0, busy = 0.0;
                for (const auto &s : subs)
                {
                    const double work = static_cast<double>(s.laneCount) * std::max<long>(1, s.tileCount * s.contrCount);
                    all += work;
                    busy += work * std::min<long>(nt / 64, (static_cast<long>(nb) * s.laneCount + 63) / 64);
                }
                const double waves = groups * (all > 0.0 ? busy / all : nt / 64.0);
                return std::sqrt(std::min(1.0, waves / 32.0));
            };
            for (auto &st : stores) st.inLds = st.wantLds;
            const double idle = utilisation(NB, NT);
            const double base = idle * occupancy(NB, NT);
            double best = base;
            int bestNB = NB, bestNT = NT;
            // Candidates: up to 16 entries per workgroup.  Kernels that carry at most a quarter of the arithmetic may
            // need several passes (a wide but cheap pointwise kernel should not dictate one entry per workgroup to
            // the narrow, expensive contractions around it); looping the contractions themselves measured slower
            // (p=3 mass apply with 12 entries in 128 lanes: 62.5 % against 76.7 %).  Never smaller workgroups than the
            // default, and everything that wants LDS must still fit.
            for (int nt : {128, 256})
            {
                if (nt < NT) continue;
                for (int nb = 1; nb <= 16 && nb <= E; ++nb)
                {
                    if (nb * maxLane > 8L * nt || multiPassShare(nb, nt) > 0.25) break;
                    if (PlaceLds(nb) > 64 * 1024 / 8) break;
                    const double u = utilisation(nb, nt) * occupancy(nb, nt);
                    if (u > best * 1.02)
                    {
                        best = u;
                        bestNB = nb;
                        bestNT = nt;
                    }
                }
            }
            // A workgroup with one batch entry and at least half of its lanes busy keeps it: the batch index is then
            // uniform, so its share of the address arithmetic is scalar, which measured no worse than fuller
            // wavefronts (p=2 mass assembly).  Groups that batch anyway take the better packing (p=1 mass apply:
            // 8 -> 14 entries per workgroup, 62.9 -> 74.9 % of the HBM peak; p=4: 2 -> 5 entries in 256 lanes,
            // 67.5 -> 72.0 %), and so do groups whose wavefronts would be mostly idle.
            const bool wanted = envInt("ACRO_HIP_PACK") > 0 || (envInt("ACRO_HIP_PACK") == 0 && (NB > 1 || idle < 0.5));
            if (wanted && best >= 1.1 * base)
            {
                NB = bestNB;
                NT = bestNT;
            }
            busyLanes = utilisation(NB, NT);
        }

        // A streaming group (one phase, nothing in LDS) whose workgroups move very little is bound by the rate at
        // which workgroups start, not by memory: with 1 - 2 KB per workgroup a copy reaches 72 % of the HBM peak and
        // an outer product 64 %.  Such groups take more batch entries per workgroup, in several passes of its lanes,
        // until a workgroup moves 8 KB (copy 72 -> 79 %, outer product 64 -> 88 %, batched 8 x 8 transpose 70 -> 77 %,
        // batched dot product 71 -> 76 %).  From 3 KB per workgroup on the same change measured slower
        // (`A_e_i += B_e_i` 77 -> 75 %, three-operand product 78 -> 75 %), hence the threshold.
        lightWorkgroups = false;
        if (opt.force_nb <= 0 && opt.force_nt <= 0 && envInt("ACRO_HIP_NB") <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0 &&
            envInt("ACRO_HIP_LIGHT") >= 0)
        {
            bool streaming = subs.back().phase == 0;
            for (const auto &st : stores) streaming = streaming && !st.wantLds && !st.staged;
            bool shared = false;   // outputs shared by lanes: their workgroups keep 128 lanes (batched dot product with
                                   // 16 entries per workgroup: 76 % in 128 lanes, 66 % in 256)
            for (const auto &s : subs)
            {
                streaming = streaming && (!s.loopMode || s.splitLanes != 0) && s.matrixOp == 0 && has(s.out.idx, batch);
                shared = shared || s.splitLanes != 0;
            }
            double perEntry = 0.0;
            std::set<int> counted;
            for (const auto &s : subs)
            {
                for (const auto &v : s.in)
                {
                    if (has(v.idx, batch) && counted.insert(v.uvar).second) perEntry += 8.0 * static_cast<double>(v.size) / static_cast<double>(E);
                }
                const double written = 8.0 * static_cast<double>(s.out.size) / static_cast<double>(E);
                if (s.op != '=' && !counted.count(s.out.uvar)) perEntry += written;  // the old value is read first
                if (counted.insert(s.out.uvar).second) perEntry += written;
            }
            if (streaming && perEntry > 0.0 && NB * perEntry < 2560.0)
            {
                long nb = NB;
                while (nb * perEntry < 8192.0 && nb * 2 <= E && nb < 256) nb *= 2;
                if (nb > NB)
                {
                    NB = static_cast<int>(nb);
                    if (static_cast<long>(NB) * maxLane >= 512 && !shared) NT = std::max(NT, 256);
                    lightWorkgroups = true;
                }
            }
        }

        // Everything that wants LDS gets it while the workgroup stays within the 64 KB a workgroup may declare
        // statically; otherwise shrink the batch, and finally leave the largest tiles in device memory.
        const int budgetDoubles = 64 * 1024 / 8;
        for (auto &st : stores) st.inLds = st.wantLds;
        // An operand staged in LDS is copied once per workgroup: the workgroup must serve enough batch entries for
        // that copy to stay small against what the entries themselves move (one entry per 256 doubles staged).
        if (opt.force_nb <= 0 && envInt("ACRO_HIP_NB") <= 0 && batch >= 0)
        {
            long staged = 0;
            for (const auto &st : stores) staged += (st.staged && st.inLds) ? uvars[st.members[0]].size : 0;
            const long wanted = std::min<long>(std::min<long>(E, 32), (staged + 255) / 256);
            if (wanted > NB)
            {
                NB = static_cast<int>(wanted);
                if (static_cast<long>(NB) * maxLane > 2L * NT) NT = 256;
            }
        }
        while (true)
        {
            ldsDoubles = PlaceLds(NB);
            if (ldsDoubles <= budgetDoubles) break;
            bool dropped = false;  // staged operands are the first to go back to device memory
            for (auto &st : stores)
            {
                if (st.staged && st.inLds && !dropped)
                {
                    st.inLds = false;
                    dropped = true;
                }
            }
            if (dropped) continue;
            if (NB > 1 && opt.force_nb <= 0)
            {
                NB /= 2;
                continue;
            }
            int biggest = -1;
            for (size_t si = 0; si < stores.size(); ++si)
            {
                if (stores[si].inLds && (biggest < 0 || stores[si].tileSize > stores[biggest].tileSize))
                    biggest = static_cast<int>(si);
            }
            if (biggest < 0) break;
            stores[biggest].inLds = false;
        }

        // Stores to device memory that may be dropped: every view of the tensor is transient, and every read of it
        // inside the group (operands and old values of += / -=) is served from registers or from the LDS tile.
        const int K = static_cast<int>(subs.size());
        for (size_t si = 0; si < stores.size(); ++si)
        {
            Storage &st = stores[si];
            st.elide = false;
            if (!st.transient || !st.written) continue;
            bool ok = true, anyRead = false;
            for (int k = 0; k < K; ++k)
            {
                const Sub &s = subs[k];
                for (size_t v = 0; v < s.in.size(); ++v)
                {
                    if (uvars[s.in[v].uvar].storage != static_cast<int>(si)) continue;
                    anyRead = true;
                    if (FromRegisters(k, static_cast<int>(v))) continue;
                    if (!(st.inLds && readCovered[k][v])) ok = false;
                }
                if (uvars[s.out.uvar].storage == static_cast<int>(si) && s.op != '=' && !s.forwardedOld)
                {
                    if (!(st.inLds && oldCovered[k])) ok = false;
                }
            }
            st.elide = ok && anyRead;
        }
        if (envInt("ACRO_HIP_LDS_PAD") > 0) PadLdsTiles(budgetDoubles);  // opt-in: see PadLdsTiles

        // A launch that writes several times what it reads streams better with fewer workgroups resident per CU
        // (fewer write streams interleave at the memory controllers): workgroups of 128 lanes become 256 lanes with
        // the upper half idle, which halves the residency.  Measured: p=2 mass assembly 37.2 -> 34.3 us, p=3 mass
        // apply with all intermediates stored 355 -> 335 us; the same change costs the read-dominated p=3 mass
        // apply with transient intermediates 8 % (86.4 -> 93.6 us), hence the condition.
        if (NT == 128 && !lightWorkgroups && opt.force_nt <= 0 && envInt("ACRO_HIP_NT") <= 0 && batch >= 0)
        {
            double stored = 0.0, loaded = 0.0;
            std::set<int> counted;
            for (int k = 0; k < K; ++k)
            {
                const Sub &s = subs[k];
                if (StoresToGlobal(k)) stored += static_cast<double>(s.out.size) / static_cast<double>(E);
                for (size_t v = 0; v < s.in.size(); ++v)
                {
                    const Source src = SourceOf(k, static_cast<int>(v));
                    if ((src == kFromGlobal || src == kFromConstant) && has(s.in[v].idx, batch) &&
                        counted.insert(s.in[v].uvar).second)
                        loaded += static_cast<double>(s.in[v].size) / static_cast<double>(E);
                }
            }
            if (stored >= 3.0 * loaded && stored > 0.0)
            {
                NT = 256;
                // Results that leave through their LDS tiles are written as one contiguous range per tensor and
                // workgroup.  Twice the batch entries in workgroups of twice the lanes keep as many entries in flight
                // per CU and make those ranges twice as long (p=3 mass apply with all intermediates stored, 4 entries
                // in 256 lanes -> 8 in 512: 336 -> 311 us; 8 in 256 lanes 332 us, 16 in 1 024 lanes 331 us).
                bool throughLds = false;
                for (int k = 0; k < K; ++k) throughLds = throughLds || CopiesOutFromLds(k);
                if (throughLds && NB >= 2 && opt.force_nb <= 0 && envInt("ACRO_HIP_NB") <= 0 && 2L * NB <= E && envInt("ACRO_HIP_WRITE_BATCH") >= 0)
                {
                    const int wider = PlaceLds(2 * NB);
                    if (wider <= budgetDoubles / 2)
                    {
                        NB *= 2;
                        NT = 512;
                        ldsDoubles = wider;
                    }
                    else
                    {
                        ldsDoubles = PlaceLds(NB);
                    }
                }
            }
        }
    }

    // ----------------------------------------------------------------------------- LDS bank conflicts
    // LDS has 64 banks of 4 bytes; a wavefront's 8-byte accesses are served 32 lanes at a time, and lanes of such a
    // group that hit the same bank at different addresses serialise.  All addresses are known here (lane index
    // decomposition, tile strides), so the cost of every LDS access instruction can be counted and the tile strides
    // padded until the count stops improving.  The count models 8-byte accesses only (the compiler merges adjacent
    // ones into 16-byte accesses).  Padding is opt-in (ACRO_HIP_LDS_PAD=1): it changed nothing measurable for the
    // p=3 mass apply, and on the p=7 diffusion chain a few hundred bytes of padding cost a resident workgroup (LDS is
    // handed out in granules) and 20 % of the speed until the acceptance test counted in granules.

    // Serialisation cycles of one access instruction whose lane l of the chain's item w reads `base(w)` doubles.
    static long ConflictCycles(const std::vector<long> &addr)
    {
        long cycles = 0;
        for (size_t g = 0; g < addr.size(); g += 32)
        {
            // distinct addresses per bank (a double covers two consecutive 4-byte banks: bank pair = addr mod 32)
            std::map<long, std::set<long>> perBank;
            for (size_t l = g; l < std::min(addr.size(), g + 32); ++l) perBank[((addr[l] % 32) + 32) % 32].insert(addr[l]);
            size_t worst = 1;
            for (const auto &b : perBank) worst = std::max(worst, b.second.size());
            cycles += static_cast<long>(worst);
        }
        return cycles;
    }

    // Lane part of the LDS address of an occurrence for every work item of its kernel.
    std::vector<long> LaneAddresses(const Sub &s, const VarRef &r, int nb) const
    {
        const Storage &st = StoreOf(r.uvar);
        const long items = static_cast<long>(nb) * s.laneCount;
        std::vector<long> addr(items);
        for (long w = 0; w < items; ++w)
        {
            const long b = w / s.laneCount;
            long rest = w % s.laneCount;
            std::vector<int> value(nidx, 0);
            for (int j = static_cast<int>(s.lane.size()) - 1; j >= 0; --j)
            {
                value[s.lane[j]] = static_cast<int>(rest % extent[s.lane[j]]);
                rest /= extent[s.lane[j]];
            }
            long a = b * st.tileSize;
            for (size_t d = 0; d < r.idx.size(); ++d)
            {
                if (r.idx[d] != batch && has(s.lane, r.idx[d])) a += static_cast<long>(value[r.idx[d]]) * LdsStride(r.uvar, d);
            }
            addr[w] = a;
        }
        return addr;
    }

    long LdsCostOfStorage(int si, int nb) const
    {
        long cost = 0;
        for (int k = 0; k < static_cast<int>(subs.size()); ++k)
        {
            const Sub &s = subs[k];
            if (s.loopMode) continue;
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (uvars[s.in[v].uvar].storage != si || SourceOf(k, static_cast<int>(v)) != kFromLds) continue;
                std::set<int> seen;
                long ninstr = 1;
                for (int id : s.in[v].idx)
                {
                    if ((has(s.tile, id) || has(s.contr, id)) && seen.insert(id).second) ninstr *= extent[id];
                }
                cost += ninstr * ConflictCycles(LaneAddresses(s, s.in[v], nb));
            }
            if (uvars[s.out.uvar].storage == si && (NeedsLdsCopy(k) || (s.op != '=' && !s.forwardedOld && OldValueInLds(k))))
                cost += s.tileCount * ConflictCycles(LaneAddresses(s, s.out, nb));
        }
        return cost;
    }

    void SetLdsStrides(Storage &st, const std::vector<int> &pad, int padEntry) const
    {
        long run = 1;
        st.ldsStride.assign(st.dims.size(), 0);
        int p = 0;
        for (int d = static_cast<int>(st.dims.size()) - 1; d >= 0; --d)
        {
            if (d == st.batchDim) continue;
            st.ldsStride[d] = static_cast<int>(run);
            run = run * st.dims[d] + pad[p++];
        }
        st.tileSize = static_cast<int>(run + padEntry);
    }

    void PadLdsTiles(int budgetDoubles)
    {
        // Padding must not cost a resident workgroup: a CU has 160 KB of LDS, handed out in granules of 1 280 bytes
        // (the p=7 diffusion chain at 53 440 bytes fits three times, at 54 080 bytes only twice).
        auto resident = [](long doubles) {
            const long bytes = (std::max<long>(1, doubles) * 8 + 1279) / 1280 * 1280;
            return 160L * 1024 / bytes;
        };
        const long residentBefore = resident(PlaceLds(NB));
        for (size_t si = 0; si < stores.size(); ++si)
        {
            Storage &st = stores[si];
            if (!st.inLds || st.staged) continue;
            const int ndim = static_cast<int>(st.dims.size()) - 1;
            std::vector<int> pad(ndim, 0), bestPad(ndim, 0);
            int bestEntry = 0;
            SetLdsStrides(st, pad, 0);
            long best = LdsCostOfStorage(static_cast<int>(si), NB);
            const long unpadded = best;
            // coordinate descent: one stride at a time, innermost first, two sweeps
            for (int sweep = 0; sweep < 2 && best > 0; ++sweep)
            {
                for (int p = 0; p <= ndim; ++p)
                {
                    const int limit = p == ndim ? 16 : 8;
                    for (int cand = 0; cand <= limit; ++cand)
                    {
                        std::vector<int> trial = bestPad;
                        int trialEntry = bestEntry;
                        if (p == ndim)
                            trialEntry = cand;
                        else
                            trial[p] = cand;
                        SetLdsStrides(st, trial, trialEntry);
                        const long c = LdsCostOfStorage(static_cast<int>(si), NB);
                        if (c < best)
                        {
                            best = c;
                            bestPad = trial;
                            bestEntry = trialEntry;
                        }
                    }
                }
            }
            SetLdsStrides(st, bestPad, bestEntry);
            const int total = PlaceLds(NB);
            if (total > budgetDoubles || best >= unpadded || (envInt("ACRO_HIP_LDS_PAD") < 2 && resident(total) < residentBefore))
            {
                SetLdsStrides(st, std::vector<int>(ndim, 0), 0);  // no room or no gain: natural layout
            }
        }
        ldsDoubles = PlaceLds(NB);
    }

    // --------------------------------------------------------------------------------------- emission
    std::ostringstream out;

    // Kernel parameters are storages; an operand addresses its storage at viewOffset.
    std::string PtrName(int uvar) const { return "T" + str(uvars[uvar].storage); }
    // Pair number of an operand that is read through an index map instead of from its own memory, or -1.
    int GatherSlot(int uvar) const
    {
        return static_cast<size_t>(uvar) < opt.gathered.size() ? opt.gathered[uvar] : -1;
    }
    int NumGatherSlots() const
    {
        int n = 0;
        for (int g : opt.gathered) n = std::max(n, g + 1);
        return n;
    }
    // Read of entry `offset` of an operand from device memory.
    std::string GlobalRead(int uvar, const std::string &offset) const
    {
        const int g = GatherSlot(uvar);
        if (g < 0) return PtrName(uvar) + "[" + offset + "]";
        return "G" + str(g) + "s[G" + str(g) + "m[" + offset + "]]";
    }
    std::string ConstPtrName(int uvar) const { return "C" + str(uvars[uvar].storage); }
    const Storage &StoreOf(int uvar) const { return stores[uvars[uvar].storage]; }
    // LDS stride of a view dimension, and the constant LDS offset of the view inside the storage's tile
    int LdsStride(int uvar, size_t d) const
    {
        const UVarInfo &op = uvars[uvar];
        return StoreOf(uvar).ldsStride[d + op.fixed.size()];
    }
    long LdsViewOffset(int uvar) const
    {
        const UVarInfo &op = uvars[uvar];
        long off = 0;
        for (size_t d = 0; d < op.fixed.size(); ++d) off += static_cast<long>(op.fixed[d]) * StoreOf(uvar).ldsStride[d];
        return off;
    }
    std::string IdxVar(int id) const { return "i_" + idxName[id]; }

    // Offset of an occurrence split into a run-time part (batch entry + lane indices) and, for a given
    // assignment of tile / contraction indices, a literal part.
    std::string RuntimeOffset(const VarRef &r, const Sub &s, bool lds) const
    {
        const UVarInfo &u = uvars[r.uvar];
        const Storage &st = StoreOf(r.uvar);
        std::string expr;
        auto add = [&](const std::string &term) { expr += (expr.empty() ? "" : " + ") + term; };
        if (lds && st.staged)
            add(str(st.ldsOffset + LdsViewOffset(r.uvar)));
        else if (lds)
            add(str(st.ldsOffset + LdsViewOffset(r.uvar)) + " + b * " + str(st.tileSize));
        else if (u.viewOffset != 0)
            add(Lit(u.viewOffset));
        // Total stride of every lane index in this occurrence (an index may occur in two dimensions).
        std::vector<long> laneStride(s.lane.size(), 0);
        for (size_t d = 0; d < r.idx.size(); ++d)
        {
            const int id = r.idx[d];
            const long stride = lds ? LdsStride(r.uvar, d) : r.stride[d];
            if (id == batch)
            {
                if (!lds) add("e * " + Lit(stride));
                continue;
            }
            for (size_t j = 0; j < s.lane.size(); ++j)
            {
                if (s.lane[j] == id) laneStride[j] += stride;
            }
        }
        // The work-item header splits the item number r_ into the lane indices, the last one fastest.  A run of
        // consecutive lane indices that this occurrence lays out the same way (the stride of one is the stride of the
        // next times its extent) needs no splitting: its terms add up to a single quotient of r_ times the last
        // stride, and for an operand that follows the lanes' order throughout the offset is r_ times a constant.
        // That spares the integer divisions and multiplications of every index in the run.
        std::vector<long> divisor(s.lane.size(), 1);  // r_ / divisor[j] % extent = lane index j
        {
            long st = s.laneCount;
            for (size_t j = 0; j < s.lane.size(); ++j)
            {
                st /= extent[s.lane[j]];
                divisor[j] = st;
            }
        }
        const bool collapse = envInt("ACRO_HIP_COLLAPSE") >= 0;
        for (size_t j = 0; j < s.lane.size();)
        {
            if (laneStride[j] == 0)
            {
                ++j;
                continue;
            }
            size_t k = j;
            long span = extent[s.lane[j]];
            while (collapse && k + 1 < s.lane.size() && laneStride[k + 1] != 0 &&
                   laneStride[k] == laneStride[k + 1] * extent[s.lane[k + 1]])
            {
                ++k;
                span *= extent[s.lane[k]];
            }
            const std::string factor = lds ? str(laneStride[k]) : Lit(laneStride[k]);
            if (k == j)
            {
                add(IdxVar(s.lane[j]) + " * " + factor);
            }
            else
            {
                std::string q = divisor[k] == 1 ? std::string("r_") : "(r_ / " + str(divisor[k]) + ")";
                if (j > 0) q = "(" + q + " % " + str(span) + ")";
                add(q + " * " + factor);
            }
            j = k + 1;
        }
        return expr.empty() ? "0" : expr;
    }

    long LiteralOffset(const VarRef &r, const Sub &s, bool lds, const std::vector<int> &value) const
    {
        long off = 0;
        for (size_t d = 0; d < r.idx.size(); ++d)
        {
            const int id = r.idx[d];
            if (id == batch || has(s.lane, id)) continue;
            off += static_cast<long>(value[id]) * (lds ? LdsStride(r.uvar, d) : r.stride[d]);
        }
        return off;
    }

    // Where an input occurrence of kernel k is read from.
    enum Source
    {
        kFromRegisters,
        kFromConstant,
        kFromLds,
        kFromGlobal
    };
    Source SourceOf(int k, int v) const
    {
        const Sub &s = subs[k];
        const VarRef &r = s.in[v];
        if (FromRegisters(k, v)) return kFromRegisters;
        if (StoreOf(r.uvar).inLds && (readCovered[k][v] || StoreOf(r.uvar).staged)) return kFromLds;
        if (IsUniform(s, r, s.tile)) return kFromConstant;
        return kFromGlobal;
    }

    // Batch part of a scalar operand's address ("e0 * stride + ", e0 being uniform) or nothing.
    std::string ScalarBase(const VarRef &r) const
    {
        std::string base;
        for (size_t d = 0; d < r.idx.size(); ++d)
        {
            if (r.idx[d] == batch) base += "e0 * " + Lit(r.stride[d]) + " + ";
        }
        return base;
    }

    // Results that the kernels of a chain have left in registers: (operand, literal offset) -> register name.
    typedef std::map<std::pair<int, long>, std::string> ForwardMap;

    struct Body
    {
        std::vector<std::string> bases;    // run-time base offsets
        std::vector<std::string> loads;    // operand loads
        std::vector<std::string> compute;  // partial sums and outputs
        std::vector<std::string> stores;
        std::map<std::string, std::string> loadMemo;
        std::map<std::string, std::string> sumMemo;
        int counter = 0;
        // Loads of per-entry pure inputs from device memory, in order of first use: (memo key, right-hand side).
        // They are what a prefetch at kernel entry would issue.
        std::vector<std::pair<std::string, std::string>> globalLoads;
    };

    // Device-memory operand that a phase may load long before it is used: never written by the group and
    // addressed through the batch index (the streaming inputs, not small tables).
    bool Prefetchable(int k, int v) const
    {
        const VarRef &r = subs[k].in[v];
        return SourceOf(k, v) == kFromGlobal && IsPureInput(r.uvar) && has(r.idx, batch);
    }

    std::string OperandExpr(int k, int v, const std::vector<int> &value, Body &body,
                            const ForwardMap &forwarded)
    {
        const Sub &s = subs[k];
        const VarRef &r = s.in[v];
        const Source src = SourceOf(k, v);
        const std::string tag = "k" + str(k) + "v" + str(v);
        if (src == kFromRegisters)
        {
            // Same work item as the producer's: the literal part of the offset names the value.
            if (s.matrixOp == 2 && r.uvar != subs[k - 1].out.uvar) return "det" + str(k - 1);
            return forwarded.at(std::make_pair(r.uvar, LiteralOffset(r, s, false, value)));
        }
        if (src == kFromConstant)
        {
            return ConstPtrName(r.uvar) + "[" + ScalarBase(r) + Lit(uvars[r.uvar].viewOffset + LiteralOffset(r, s, false, value)) + "]";
        }
        const bool lds = (src == kFromLds);
        const long off = LiteralOffset(r, s, lds, value);
        const std::string key = tag + ":" + str(off);
        auto it = body.loadMemo.find(key);
        if (it != body.loadMemo.end()) return it->second;
        const std::string name = "x" + str(k) + "_" + str(body.counter++);
        const std::string base = "o_" + tag;
        if (lds)
        {
            body.loads.push_back("const double " + name + " = lds[" + base + " + " + str(off) + "];");
        }
        else
        {
            const std::string rhs = GlobalRead(r.uvar, base + " + " + Lit(off));
            body.loads.push_back("const double " + name + " = " + rhs + ";");
            if (Prefetchable(k, v)) body.globalLoads.push_back(std::make_pair(key, rhs));
        }
        body.loadMemo[key] = name;
        return name;
    }

    // Sum over the contraction indices deeper than `depth`, of the product of the factors that close at those
    // levels.  Returns the name of a temporary, or "" when the remaining sum is exactly one.
    std::string PartialSum(int k, int depth, std::vector<int> &value, Body &body, const std::vector<int> &level,
                           const ForwardMap &forwarded)
    {
        const Sub &s = subs[k];
        const int n = static_cast<int>(s.contr.size());
        if (depth == n) return "";

        // The value depends on the already assigned indices only through the deeper factors.
        std::set<int> relevant;
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            if (level[v] > depth)
            {
                for (int id : s.in[v].idx)
                {
                    if (id != batch && !has(s.lane, id)) relevant.insert(id);
                }
            }
        }
        std::string key = "d" + str(depth);
        for (int id : relevant)
        {
            bool assigned = has(s.tile, id);
            for (int j = 0; j < depth; ++j) assigned = assigned || s.contr[j] == id;
            if (assigned) key += "," + str(id) + "=" + str(value[id]);
        }
        auto it = body.sumMemo.find(key);
        if (it != body.sumMemo.end()) return it->second;

        const int cid = s.contr[depth];
        std::vector<std::string> terms;
        for (int x = 0; x < extent[cid]; ++x)
        {
            value[cid] = x;
            std::string prod;
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (level[v] != depth + 1) continue;
                const std::string opnd = OperandExpr(k, static_cast<int>(v), value, body, forwarded);
                prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
            }
            const std::string rest = PartialSum(k, depth + 1, value, body, level, forwarded);
            std::string term;
            if (prod.empty() && rest.empty())
                term = "1.0";
            else if (prod.empty())
                term = rest;
            else if (rest.empty())
                term = prod;
            else
                term = prod + " * " + rest;
            terms.push_back(term);
        }
        value[cid] = 0;
        const std::string name = "s" + str(k) + "_" + str(body.counter++);
        body.compute.push_back("double " + name + " = " + terms[0] + ";");
        for (size_t t = 1; t < terms.size(); ++t) body.compute.push_back(name + " += " + terms[t] + ";");
        body.sumMemo[key] = name;
        return name;
    }

    void EmitBases(int k, Body &body)
    {
        const Sub &s = subs[k];
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            const Source src = SourceOf(k, static_cast<int>(v));
            if (src == kFromRegisters || src == kFromConstant) continue;
            body.bases.push_back(std::string("const ") + (src == kFromLds ? "int" : OffsetType()) + " o_k" + str(k) + "v" +
                                 str(v) + " = " + RuntimeOffset(s.in[v], s, src == kFromLds) + ";");
        }
        body.bases.push_back(std::string("const ") + OffsetType() + " o_k" + str(k) + "g = " + RuntimeOffset(s.out, s, false) + ";");
        if (StoreOf(s.out.uvar).inLds)
            body.bases.push_back("const int o_k" + str(k) + "l = " + RuntimeOffset(s.out, s, true) + ";");
    }

    // Is the output variable's tile already on chip before kernel k (needed by += and -=)?
    bool OldValueInLds(int k) const { return StoreOf(subs[k].out.uvar).inLds && oldCovered[k]; }

    // The store of kernel k's output to device memory is dead when a later kernel of the group rewrites the same
    // view completely, takes the old value from the LDS tile (or does not need it), and every read in between is
    // served from the tile as well.
    bool StoreIsDead(int k) const
    {
        const int outVar = subs[k].out.uvar;
        const Storage &st = StoreOf(outVar);
        if (subs[k].out.repeated) return false;
        const bool nextTakesRegisters = k + 1 < static_cast<int>(subs.size()) && subs[k + 1].forwardedOld;
        if (!st.inLds && !nextTakesRegisters) return false;
        const int si = uvars[outVar].storage;
        for (int j = k + 1; j < static_cast<int>(subs.size()); ++j)
        {
            const Sub &s = subs[j];
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (uvars[s.in[v].uvar].storage != si) continue;
                if (!FromRegisters(j, static_cast<int>(v)) && !(st.inLds && readCovered[j][v])) return false;
            }
            if (uvars[s.out.uvar].storage == si && s.out.uvar != outVar) return false;  // keep it simple: same view only
            if (s.out.uvar == outVar) return s.op == '=' || s.forwardedOld || (st.inLds && oldCovered[j]);
        }
        return false;
    }

    bool StoresToGlobal(int k) const { return !StoreOf(subs[k].out.uvar).elide && !StoreIsDead(k); }

    // A result that no later kernel of the launch reads back from device memory is written with a non-temporal
    // store: it streams to HBM without displacing the operands that the strided loads of other lanes still need in
    // the caches (measured +2.5 % on the p=3 mass apply; non-temporal LOADS measured -20 % and are not used).
    // Such stores complete later, which delays the retirement of the workgroup: where LDS allows only a few resident
    // workgroups per CU that costs more than it gains (p=7 diffusion apply, 3 workgroups per CU: -14 %), so they are
    // only used while at least 8 workgroups fit.
    // They also get less write combining, so they are only used when one store instruction of a wavefront fills at
    // least about half of every 128-byte line it touches (scattered 8-byte pieces written this way measured 1.7x
    // slower than ordinary stores).
    bool StreamsOut(int k) const
    {
        if (envInt("ACRO_HIP_NT_STORE") < 0) return false;
        if (static_cast<long>(ldsDoubles) * 8 > 20 * 1024) return false;
        if (WaveStoreLineCoverage(k) < 0.45) return false;
        const int si = uvars[subs[k].out.uvar].storage;
        for (int j = k + 1; j < static_cast<int>(subs.size()); ++j)
        {
            const Sub &s = subs[j];
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (uvars[s.in[v].uvar].storage == si && SourceOf(j, static_cast<int>(v)) == kFromGlobal) return false;
            }
            if (uvars[s.out.uvar].storage == si && s.op != '=' && !s.forwardedOld && !OldValueInLds(j)) return false;
        }
        return true;
    }

    // How much of the 128-byte lines that one store instruction of kernel k touches does it fill, on average over
    // the instructions of the first wavefront?  A lane's stores to consecutive addresses are counted as one
    // instruction per pair of doubles (the compiler merges them into 16-byte stores).
    double WaveStoreLineCoverage(int k) const
    {
        const Sub &s = subs[k];
        const long items = std::min<long>(64, static_cast<long>(NB) * s.laneCount);
        std::vector<std::vector<long>> perLane(items);
        for (long w = 0; w < items; ++w)
        {
            std::vector<int> value(nidx, 0);
            long rest = w % s.laneCount;
            for (int j = static_cast<int>(s.lane.size()) - 1; j >= 0; --j)
            {
                value[s.lane[j]] = static_cast<int>(rest % extent[s.lane[j]]);
                rest /= extent[s.lane[j]];
            }
            if (batch >= 0) value[batch] = static_cast<int>(w / s.laneCount);
            const long tiles = s.loopMode ? 1 : s.tileCount;
            for (long t = 0; t < tiles; ++t)
            {
                long rem = t;
                for (int j = static_cast<int>(s.tile.size()) - 1; j >= 0; --j)
                {
                    value[s.tile[j]] = static_cast<int>(rem % extent[s.tile[j]]);
                    rem /= extent[s.tile[j]];
                }
                long a = uvars[s.out.uvar].viewOffset;
                for (size_t d = 0; d < s.out.idx.size(); ++d) a += static_cast<long>(value[s.out.idx[d]]) * s.out.stride[d];
                perLane[w].push_back(a);
            }
            std::sort(perLane[w].begin(), perLane[w].end());
        }
        // instruction g of a lane = its g-th group of (up to two) consecutive addresses
        std::vector<std::map<long, int>> doublesPerLine;
        for (long w = 0; w < items; ++w)
        {
            size_t g = 0;
            for (size_t i = 0; i < perLane[w].size(); ++g)
            {
                const size_t n = (i + 1 < perLane[w].size() && perLane[w][i + 1] == perLane[w][i] + 1) ? 2 : 1;
                if (doublesPerLine.size() <= g) doublesPerLine.resize(g + 1);
                for (size_t j = 0; j < n; ++j) doublesPerLine[g][perLane[w][i + j] / 16] += 1;
                i += n;
            }
        }
        double sum = 0.0;
        long lines = 0;
        for (const auto &instr : doublesPerLine)
        {
            for (const auto &l : instr)
            {
                sum += std::min(16, l.second) / 16.0;
                ++lines;
            }
        }
        return lines == 0 ? 0.0 : sum / static_cast<double>(lines);
    }

    std::string GlobalStore(int k, const std::string &gaddr, const std::string &value) const
    {
        if (StreamsOut(k)) return "__builtin_nontemporal_store(" + value + ", &" + gaddr + ");";
        return gaddr + " = " + value + ";";
    }

    bool NeedsLdsCopy(int k) const
    {
        const Storage &st = StoreOf(subs[k].out.uvar);
        return st.inLds && (st.liveTo > k || st.copyOutOnly);
    }

    // A result that must reach device memory AND stays in LDS for a later kernel is written to device memory from
    // the LDS tiles, by the whole workgroup, right after the barrier that ends its phase: the tiles of a workgroup's
    // batch entries are one contiguous range of the tensor, so every store instruction of a wavefront writes 512
    // contiguous bytes, where the lanes' own stores are pencils (a few doubles per lane at a stride).  Needs the
    // tensor to carry the batch index first, the kernel to be the only writer of the whole tensor in the group, and
    // the natural (unpadded) tile layout.
    bool CopiesOutFromLds(int k) const
    {
        if (envInt("ACRO_HIP_LDS_COPY_OUT") < 0 || envInt("ACRO_HIP_PERSIST") > 0 || envInt("ACRO_HIP_LDS_PAD") > 0) return false;
        const Sub &s = subs[k];
        if (!NeedsLdsCopy(k) || !StoresToGlobal(k) || s.out.repeated) return false;
        const UVarInfo &u = uvars[s.out.uvar];
        const Storage &st = stores[u.storage];
        // the copy runs after the barrier that ends the phase: the last phase has one only for a tile kept for this
        if (s.phase == subs.back().phase && !st.copyOutOnly) return false;
        if (st.members.size() != 1 || st.batchDim != 0 || !u.fixed.empty() || u.viewOffset != 0) return false;
        for (size_t j = 0; j < subs.size(); ++j)
        {
            if (static_cast<int>(j) != k && uvars[subs[j].out.uvar].storage == u.storage) return false;
        }
        return true;
    }

    // Unrolled body of kernel k for one work item.  `forwarded` maps the literal output offsets of the previous
    // kernel to the registers holding them; on return it describes this kernel's outputs.
    void EmitUnrolledBody(int k, ForwardMap &forwarded, std::vector<std::string> &lines,
                          const std::map<std::string, std::string> *preloaded = nullptr,
                          std::vector<std::pair<std::string, std::string>> *globalLoads = nullptr)
    {
        const Sub &s = subs[k];
        Body body;
        if (preloaded != nullptr) body.loadMemo = *preloaded;
        EmitBases(k, body);

        const int n = static_cast<int>(s.contr.size());
        std::vector<int> level(s.in.size(), 0);
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            for (int j = 0; j < n; ++j)
            {
                if (has(s.in[v].idx, s.contr[j])) level[v] = j + 1;
            }
        }

        if (s.matrixOp != 0)
        {
            EmitMatrixBody(k, body, forwarded);
            // no multiply-add fusion: the results are bit-identical to the host formulas, as those of the precompiled
            // batched matrix kernels are
            lines.push_back("#pragma clang fp contract(off)");
            lines.push_back("// " + s.text + (s.matrixOp == 1 ? "   (matrix inverse)" : "   (determinant)"));
            for (const auto &l : body.bases) lines.push_back(l);
            for (const auto &l : body.loads) lines.push_back(l);
            for (const auto &l : body.compute) lines.push_back(l);
            for (const auto &l : body.stores) lines.push_back(l);
            if (globalLoads != nullptr) *globalLoads = body.globalLoads;
            return;
        }

        std::vector<int> value(nidx, 0);
        const long tc = s.tileCount;
        for (long t = 0; t < tc; ++t)
        {
            long rem = t;
            for (int j = static_cast<int>(s.tile.size()) - 1; j >= 0; --j)
            {
                value[s.tile[j]] = static_cast<int>(rem % extent[s.tile[j]]);
                rem /= extent[s.tile[j]];
            }
            std::string prod;
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                if (level[v] != 0) continue;
                const std::string opnd = OperandExpr(k, static_cast<int>(v), value, body, forwarded);
                prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
            }
            const std::string rest = PartialSum(k, 0, value, body, level, forwarded);
            std::string rhs;
            if (prod.empty() && rest.empty())
                rhs = "1.0";
            else if (prod.empty())
                rhs = rest;
            else if (rest.empty())
                rhs = prod;
            else
                rhs = prod + " * " + rest;

            const long goff = LiteralOffset(s.out, s, false, value);
            const long loff = StoreOf(s.out.uvar).inLds ? LiteralOffset(s.out, s, true, value) : 0;
            const std::string gaddr = PtrName(s.out.uvar) + "[o_k" + str(k) + "g + " + Lit(goff) + "]";
            const std::string laddr = "lds[o_k" + str(k) + "l + " + str(loff) + "]";
            const std::string name = "r" + str(k) + "_" + str(t);
            if (s.op == '=')
            {
                body.compute.push_back("const double " + name + " = " + rhs + ";");
            }
            else
            {
                const std::string old = s.forwardedOld ? forwarded.at(std::make_pair(s.out.uvar, goff))
                                                       : (OldValueInLds(k) ? laddr : gaddr);
                body.compute.push_back("const double " + name + " = " + old + (s.op == '+' ? " + " : " - ") + rhs + ";");
            }
            if (NeedsLdsCopy(k)) body.stores.push_back(laddr + " = " + name + ";");
            if (StoresToGlobal(k) && !CopiesOutFromLds(k)) body.stores.push_back(GlobalStore(k, gaddr, name));
            forwarded[std::make_pair(s.out.uvar, goff)] = name;
        }

        // The scope of a kernel applied after a matrix kernel is nested in that kernel's: back to the default there.
        for (int q = k; q > 0 && subs[q].fusedWithPrev; --q)
        {
            if (subs[q - 1].matrixOp == 0) continue;
            lines.push_back("#pragma clang fp contract(fast)");
            break;
        }
        lines.push_back("// " + s.text);
        for (const auto &l : body.bases) lines.push_back(l);
        for (const auto &l : body.loads) lines.push_back(l);
        for (const auto &l : body.compute) lines.push_back(l);
        for (const auto &l : body.stores) lines.push_back(l);
        if (globalLoads != nullptr) *globalLoads = body.globalLoads;
    }

    // One work item of a matrix kernel: the entries of the operand's matrix are loaded like any operand, the
    // formulas are those of the reference's host implementation (ops/NativeCPUOps.hpp:38-86), term by term in the
    // same order (the compiler may still fuse a multiply and an add): det = A0 A4 A8 + A1 A5 A6 + A2 A3 A7 - A6 A4 A2
    // - A7 A5 A0 - A8 A3 A1 (row-major entries), inverse entry (i, j) = cofactor laid out as the reference lays it
    // out, times 1.0 / det.
    void EmitMatrixBody(int k, Body &body, ForwardMap &forwarded)
    {
        const Sub &s = subs[k];
        const int n = s.matrixN;
        const VarRef &r = s.in[0];
        const int rowId = r.idx[r.idx.size() - 2], colId = r.idx[r.idx.size() - 1];
        const std::string detName = "det" + str(k);
        const bool reuse = s.matrixOp == 2 && s.fusedWithPrev && subs[k - 1].matrixOp == 1;
        std::vector<std::string> a(n * n);
        std::vector<int> value(nidx, 0);
        if (!reuse)
        {
            for (int i = 0; i < n; ++i)
            {
                for (int j = 0; j < n; ++j)
                {
                    value[rowId] = i;
                    value[colId] = j;
                    a[i * n + j] = OperandExpr(k, 0, value, body, forwarded);
                }
            }
        }
        auto mul = [](const std::string &x, const std::string &y) { return x + " * " + y; };
        if (reuse)
            body.compute.push_back("const double " + detName + " = det" + str(k - 1) + ";");
        else if (n == 1)
            body.compute.push_back("const double " + detName + " = " + a[0] + ";");
        else if (n == 2)
            body.compute.push_back("const double " + detName + " = " + mul(a[0], a[3]) + " - " + mul(a[1], a[2]) + ";");
        else
            body.compute.push_back("const double " + detName + " = " + a[0] + " * " + a[4] + " * " + a[8] + " + " + a[1] + " * " +
                                   a[5] + " * " + a[6] + " + " + a[2] + " * " + a[3] + " * " + a[7] + " - " + a[6] + " * " + a[4] +
                                   " * " + a[2] + " - " + a[7] + " * " + a[5] + " * " + a[0] + " - " + a[8] + " * " + a[3] + " * " +
                                   a[1] + ";");

        std::vector<std::string> result;  // right-hand sides in tile order (row-major entries of the output)
        if (s.matrixOp == 2)
        {
            result.push_back(detName);
        }
        else
        {
            const std::string inv = "inv" + str(k);
            body.compute.push_back("const double " + inv + " = 1.0 / " + detName + ";");
            if (n == 1)
            {
                result = {inv};
            }
            else if (n == 2)
            {
                result = {inv + " * " + a[3], "-" + inv + " * " + a[1], "-" + inv + " * " + a[2], inv + " * " + a[0]};
            }
            else
            {
                auto cof = [&](int p, int q, int u, int v) { return inv + " * (" + mul(a[p], a[q]) + " - " + mul(a[u], a[v]) + ")"; };
                result = {cof(4, 8, 5, 7), cof(5, 6, 3, 8), cof(3, 7, 4, 6), cof(2, 7, 1, 8), cof(0, 8, 2, 6),
                          cof(1, 6, 0, 7), cof(1, 5, 2, 4), cof(2, 3, 0, 5), cof(0, 4, 1, 3)};
            }
        }
        for (size_t t = 0; t < result.size(); ++t)
        {
            std::fill(value.begin(), value.end(), 0);
            if (s.matrixOp == 1)
            {
                value[s.tile[0]] = static_cast<int>(t) / n;
                value[s.tile[1]] = static_cast<int>(t) % n;
            }
            const long goff = LiteralOffset(s.out, s, false, value);
            const long loff = StoreOf(s.out.uvar).inLds ? LiteralOffset(s.out, s, true, value) : 0;
            const std::string gaddr = PtrName(s.out.uvar) + "[o_k" + str(k) + "g + " + Lit(goff) + "]";
            const std::string laddr = "lds[o_k" + str(k) + "l + " + str(loff) + "]";
            const std::string name = "r" + str(k) + "_" + str(static_cast<long>(t));
            body.compute.push_back("const double " + name + " = " + result[t] + ";");
            if (NeedsLdsCopy(k)) body.stores.push_back(laddr + " = " + name + ";");
            if (StoresToGlobal(k) && !CopiesOutFromLds(k)) body.stores.push_back(GlobalStore(k, gaddr, name));
            forwarded[std::make_pair(s.out.uvar, goff)] = name;
        }
    }

    // Counted-loop body (long contractions): one output per work item, no tile.
    // One output per batch entry, its contraction shared by s.splitLanes adjacent lanes.
    void EmitSplitLanesBody(int k, std::vector<std::string> &lines)
    {
        const Sub &s = subs[k];
        Body body;
        EmitBases(k, body);
        const int L = s.splitLanes;
        lines.push_back("// " + s.text + "   (contraction shared by " + str(L) + " lanes)");
        for (const auto &l : body.bases) lines.push_back(l);
        lines.push_back("const int cl = w & " + str(L - 1) + ";");
        lines.push_back("double sum = 0.0;");
        // eight loads in flight per lane (row sums of 1 024 terms: 69 % of the HBM peak with 4, 75 % with 8, 73 % with 16)
        lines.push_back("#pragma unroll 8");
        lines.push_back("for (int c = cl; c < " + str(s.contrCount) + "; c += " + str(L) + ")");
        lines.push_back("{");
        long st = s.contrCount;
        for (size_t j = 0; j < s.contr.size(); ++j)
        {
            st /= extent[s.contr[j]];
            const std::string name = IdxVar(s.contr[j]);
            if (s.contr.size() == 1)
                lines.push_back("    const int " + name + " = c;");
            else if (j == 0)
                lines.push_back("    const int " + name + " = c / " + str(st) + ";");
            else
                lines.push_back("    const int " + name + " = (c / " + str(st) + ") % " + str(extent[s.contr[j]]) + ";");
        }
        std::string prod;
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            const VarRef &r = s.in[v];
            const Source src = SourceOf(k, static_cast<int>(v));
            const bool lds = (src == kFromLds);
            std::string off;
            for (size_t d = 0; d < r.idx.size(); ++d)
            {
                const int id = r.idx[d];
                if (!has(s.contr, id)) continue;
                const long stride = lds ? LdsStride(r.uvar, d) : r.stride[d];
                off += (off.empty() ? "" : " + ") + IdxVar(id) + " * " + (lds ? str(stride) : Lit(stride));
            }
            if (off.empty()) off = "0";
            std::string opnd;
            if (src == kFromConstant)
                opnd = ConstPtrName(r.uvar) + "[" + ScalarBase(r) + Lit(uvars[r.uvar].viewOffset) + " + " + off + "]";
            else if (lds)
                opnd = "lds[o_k" + str(k) + "v" + str(v) + " + " + off + "]";
            else
                opnd = GlobalRead(r.uvar, "o_k" + str(k) + "v" + str(v) + " + " + off);
            prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
        }
        lines.push_back("    sum += " + prod + ";");
        lines.push_back("}");
        // The lanes of an output are adjacent and aligned, so every exchange partner works on the same output.  Lanes
        // 1 and 2 apart swap inside their quad; then every lane of a quad holds the same value and mirroring the
        // half row (8 lanes), then the row (16 lanes), pairs each quad with the one it has not met yet.  Every lane
        // ends up with the same sum, added in the same order.
        static const char *const kDppControl[4] = {"0xB1", "0x4E", "0x141", "0x140"};  // quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror, row_mirror
        for (int step = 0; (1 << step) < L; ++step)
        {
            lines.push_back("{");
            lines.push_back("    union { double d; int i[2]; } mine, other;");
            lines.push_back("    mine.d = sum;");
            lines.push_back(std::string("    other.i[0] = __builtin_amdgcn_update_dpp(0, mine.i[0], ") + kDppControl[step] + ", 0xF, 0xF, false);");
            lines.push_back(std::string("    other.i[1] = __builtin_amdgcn_update_dpp(0, mine.i[1], ") + kDppControl[step] + ", 0xF, 0xF, false);");
            lines.push_back("    sum += other.d;");
            lines.push_back("}");
        }
        const std::string gaddr = PtrName(s.out.uvar) + "[o_k" + str(k) + "g]";
        lines.push_back("if (cl == 0)");
        lines.push_back("{");
        if (s.op == '=')
            lines.push_back("    " + GlobalStore(k, gaddr, "sum"));
        else
            lines.push_back("    " + gaddr + " = " + gaddr + (s.op == '+' ? " + sum;" : " - sum;"));
        lines.push_back("}");
    }

    void EmitLoopBody(int k, std::vector<std::string> &lines)
    {
        const Sub &s = subs[k];
        if (s.splitLanes > 0)
        {
            EmitSplitLanesBody(k, lines);
            return;
        }
        Body body;
        EmitBases(k, body);
        lines.push_back("// " + s.text + "   (contraction as counted loops)");
        for (const auto &l : body.bases) lines.push_back(l);
        lines.push_back("double sum = 0.0;");
        std::string indent;
        for (size_t j = 0; j < s.contr.size(); ++j)
        {
            const std::string c = IdxVar(s.contr[j]);
            if (j + 1 == s.contr.size()) lines.push_back(indent + "#pragma unroll 4");
            lines.push_back(indent + "for (int " + c + " = 0; " + c + " < " + str(extent[s.contr[j]]) + "; ++" + c + ")");
            lines.push_back(indent + "{");
            indent += "    ";
        }
        std::string prod;
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            const VarRef &r = s.in[v];
            const Source src = SourceOf(k, static_cast<int>(v));
            const bool lds = (src == kFromLds);
            std::string off;
            for (size_t d = 0; d < r.idx.size(); ++d)
            {
                const int id = r.idx[d];
                if (!has(s.contr, id)) continue;
                const long st = lds ? LdsStride(r.uvar, d) : r.stride[d];
                off += (off.empty() ? "" : " + ") + IdxVar(id) + " * " + (lds ? str(st) : Lit(st));
            }
            if (off.empty()) off = "0";
            std::string opnd;
            if (src == kFromConstant)
                opnd = ConstPtrName(r.uvar) + "[" + ScalarBase(r) + Lit(uvars[r.uvar].viewOffset) + " + " + off + "]";
            else if (lds)
                opnd = "lds[o_k" + str(k) + "v" + str(v) + " + " + off + "]";
            else
                opnd = GlobalRead(r.uvar, "o_k" + str(k) + "v" + str(v) + " + " + off);
            prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
        }
        lines.push_back(indent + "sum += " + prod + ";");
        for (size_t j = 0; j < s.contr.size(); ++j)
        {
            indent.resize(indent.size() - 4);
            lines.push_back(indent + "}");
        }
        const std::string gaddr = PtrName(s.out.uvar) + "[o_k" + str(k) + "g]";
        const std::string laddr = "lds[o_k" + str(k) + "l]";
        if (s.op == '=')
            lines.push_back("const double r = sum;");
        else
            lines.push_back(std::string("const double r = ") + (OldValueInLds(k) ? laddr : gaddr) +
                            (s.op == '+' ? " + sum;" : " - sum;"));
        if (NeedsLdsCopy(k)) lines.push_back(laddr + " = r;");
        if (StoresToGlobal(k) && !CopiesOutFromLds(k)) lines.push_back(GlobalStore(k, gaddr, "r"));
    }

    // ------------------------------------------------------------------------------ reduction schedule
    // A single kernel with few output entries and a very long contraction ("S_i_j = A_n_i_j B_n" with n = 2^20):
    // mapping lanes to outputs would leave the device idle, so the flattened contraction range is split over
    // workgroups and over the lanes of a workgroup.  Lane (slice, output entry) accumulates a private partial sum
    // over its share, the workgroup adds its slices in LDS and writes one partial per output entry to a scratch
    // buffer, and a second, single-workgroup kernel adds the per-workgroup partials in a fixed order (no
    // floating-point atomics: results are reproducible from run to run).
    static constexpr long kReductionMinContraction = 2048;
    static constexpr long kReductionMaxOutputs = 128;
    static constexpr int kReductionLanes = 256;

    bool UseReductionSchedule() const
    {
        if (subs.size() != 1 || NumGatherSlots() > 0) return false;
        const Sub &s = subs[0];
        if (s.out.repeated) return false;
        return s.contrCount >= kReductionMinContraction && product(s.outIdx, extent) <= kReductionMaxOutputs;
    }

    // Expression for the element offset of an occurrence given variables named i_<index> for every loop index.
    std::string FullOffset(const VarRef &r) const
    {
        std::string expr = uvars[r.uvar].viewOffset != 0 ? Lit(uvars[r.uvar].viewOffset) : std::string();
        for (size_t d = 0; d < r.idx.size(); ++d)
            expr += (expr.empty() ? "" : " + ") + IdxVar(r.idx[d]) + " * " + Lit(r.stride[d]);
        return expr.empty() ? "0" : expr;
    }

    // Kernel parameters: one pointer per storage, taken from a representative member occurrence.
    // Storages that are kernel parameters: all but the intermediates of a factorised kernel, which are numbered last.
    int NumParamStores() const
    {
        int n = 0;
        for (const auto &st : stores)
        {
            if (!uvars[st.members[0]].isVirtual) ++n;
        }
        for (int si = 0; si < n; ++si) ACROBATIC_ASSERT(!uvars[stores[si].members[0]].isVirtual, "HIP generator: storage order");
        return n;
    }

    void FillParams(HipKernelPlan &plan, bool honour_elision) const
    {
        const int S = NumParamStores();
        plan.param_occurrence.resize(S);
        plan.param_offset.assign(S, 0);
        plan.stored.assign(S, false);
        for (int si = 0; si < S; ++si)
        {
            const int rep = stores[si].members[0];
            plan.param_occurrence[si] = FirstOccurrence(rep);
            plan.param_offset[si] = uvars[rep].viewOffset;
            plan.stored[si] = stores[si].written && !(honour_elision && stores[si].elide);
        }
    }

    std::string ParamList() const
    {
        std::string p;
        for (size_t si = 0; si < static_cast<size_t>(NumParamStores()); ++si)
        {
            p += std::string(si ? ", " : "") + (stores[si].written ? "double *" : "const double *") +
                 (opt.noalias ? "__restrict__ " : "") + "T" + str(static_cast<long>(si));
        }
        for (int g = 0; g < NumGatherSlots(); ++g)
            p += ", const int *__restrict__ G" + str(g) + "m, const double *__restrict__ G" + str(g) + "s";
        return p;
    }

    void EmitReduction(HipKernelPlan &plan)
    {
        const Sub &s = subs[0];
        const long O = product(s.outIdx, extent);
        const long Nc = s.contrCount;
        // Lanes follow the memory order of the largest operand: output entries fastest when its innermost
        // dimension is an output index, contraction slices fastest otherwise.
        const VarRef *big = &s.in[0];
        for (const auto &r : s.in)
        {
            if (r.size > big->size) big = &r;
        }
        const bool outputsFastest = has(s.outIdx, big->idx.back());
        // Few output entries that are the fastest dimension of the big operand ("S_i_j = A_n_i_j B_n"): a lane owns
        // whole contraction slices and keeps one accumulator per output entry ("pencil").  It reads the O entries of
        // its slice of A as 16-byte pieces and the slice's entry of B once, i.e. 6 load instructions per 80 bytes;
        // with one lane per (slice, output entry) every lane loads B again and the same bytes take 18 load
        // instructions (A alone streamed at 6.1 TB/s that way, A and B together at 5.0 - 5.5 TB/s).
        const bool pencil = outputsFastest && O <= 16 && envInt("ACRO_HIP_RED_PENCIL") >= 0;
        const int NTr = kReductionLanes;
        // Contraction index fastest and more than four outputs ("S_i = A_i_n" with 64 rows): with all outputs in every
        // workgroup only NTr / O lanes would walk along a row (32-byte pieces of 64 different rows per load
        // instruction).  Instead a workgroup takes four outputs, 64 adjacent lanes each, and the workgroups are dealt
        // out over groups of outputs as well as over the contraction range.
        const bool byRows = !pencil && !outputsFastest && O > 4 && NTr / O < 64 && envInt("ACRO_HIP_ONE_PASS") <= 0 &&
                            envInt("ACRO_HIP_RED_ROWS") >= 0;
        const long Sn = pencil ? NTr : (byRows ? 64 : NTr / O);  // contraction slices per workgroup and step
        const long Ow = NTr / Sn, Go = byRows ? (O + Ow - 1) / Ow : 1;  // outputs per workgroup, groups of outputs
        // First-stage workgroups.  Pencil: one per CU (256 on this device) without unrolling, i.e. about 20 KB of
        // loads in flight per CU and one 4.7 MB window moving through the operands; more workgroups or deeper
        // unrolling measured slower at every n (n = 2^24: 206 us with 256 workgroups, 216 with 512, 252 with 2 048;
        // 214 / 263 us with the loop unrolled 2 / 4 times).  One lane per (slice, output entry): 8 bytes per lane
        // and load, so up to 512 workgroups and four loads in flight per lane (also swept: 256 - 8 192 workgroups,
        // unroll 1 - 8).
        const long G = byRows ? std::min<long>(std::max<long>(1, 1024 / Go), std::max<long>(1, Nc / (Sn * 16)))
                              : std::min<long>(pencil ? 256 : 512, std::max<long>(1, Nc / (Sn * (pencil ? 4 : 16))));
        // G counts the shares of the contraction range (rows of partials in the scratch buffer); the grid has one
        // workgroup per share and group of outputs.
        const long gridG = G * Go;
        // Lanes of the finishing kernel: enough for every lane to have all its loads of partials in flight at once
        // (the kernel is a chain of memory latencies: launch, one round of loads, LDS; 1024 lanes instead of 256
        // measured 16.8 instead of 17.2 us for the pair of launches at n = 2^20), at most 1024.  The one-pass
        // variant finishes with the lanes of the partial kernel.
        int NTf = NTr;
        if (envInt("ACRO_HIP_ONE_PASS") <= 0)
        {
            NTf = kReductionLanes;
            while (NTf < 1024 && G * O > NTf * 4) NTf *= 2;
        }
        const long S2 = NTf / O;

        const std::string dimName = mk.GetDimensionedNameString();
        char hex[32];
        std::snprintf(hex, sizeof(hex), "%016llx",
                      static_cast<unsigned long long>(hashString(dimName + "/reduction/" + (opt.noalias ? "n" : "a") +
                                                                 (Positional() ? "p" : "u") +
                                                                 (envInt("ACRO_HIP_ONE_PASS") <= 0 ? "2" : (envInt("ACRO_HIP_ONE_PASS") >= 2 ? "1l" : "1")) + "/" + str(envInt("ACRO_HIP_RED_PENCIL")) +
                                                                 (byRows ? "/rows" : ""))));
        plan.module_name = std::string("acro_red_") + hex;
        const std::string fPartial = plan.module_name + "_partial", fFinal = plan.module_name + "_final";

        std::ostringstream sched;
        sched << "reduction schedule: " << O << " output entries, contraction of " << Nc << " terms split over " << G
              << " workgroups x " << Sn << " slices ("
              << (pencil ? "a lane owns whole slices"
                         : (byRows ? "four outputs per workgroup, 64 adjacent lanes along each"
                                   : (outputsFastest ? "output entries on adjacent lanes" : "slices on adjacent lanes")))
              << "), partials added in a fixed order by "
              << (envInt("ACRO_HIP_ONE_PASS") <= 0 ? "a second kernel" : "the workgroup that finishes last") << "\n  [0] " << s.text << "\n";
        plan.schedule = sched.str();

        out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
        {
            std::istringstream lines(plan.schedule);
            std::string l;
            while (std::getline(lines, l)) out << "// " << l << "\n";
        }
        auto decompose = [&](const std::vector<int> &ids, const std::string &flat, const std::string &indent) {
            long st = product(ids, extent);
            for (size_t j = 0; j < ids.size(); ++j)
            {
                st /= extent[ids[j]];
                out << indent << "const int " << IdxVar(ids[j]) << " = (int)(";
                if (j == 0)
                    out << flat << " / " << st;
                else
                    out << "(" << flat << " / " << st << ") % " << extent[ids[j]];
                out << ");\n";
            }
        };

        const bool twoKernels = envInt("ACRO_HIP_ONE_PASS") <= 0;
        const std::string counter = "(unsigned int *)(scratch + " + str(G * O) + ")";

        // ---- stage 1: per-workgroup partial sums
        out << "\nextern \"C\" __global__ __launch_bounds__(" << NTr << ") void " << fPartial << "(" << ParamList()
            << ", double *__restrict__ scratch)\n{\n";
        out << "    __shared__ double red[" << (pencil ? NTr * O : (byRows ? NTr + Ow * 16 : NTr)) << "];\n";
        if (!twoKernels) out << "    __shared__ int isLast;\n";
        out << "    const int lane = threadIdx.x;\n";
        // Workgroups interleave: in every step the G workgroups together read one contiguous window of the
        // operands, so the device-wide access pattern is a single moving front.  Neighbouring workgroups share the
        // cache lines at their border, so neighbours run on the same XCD (one L2): hardware deals consecutive
        // workgroup ids round-robin to the 8 XCDs.
        const std::string gExpr = (G % 8 == 0) ? "(long)(blockIdx.x % 8) * " + str(G / 8) + " + blockIdx.x / 8" : std::string("blockIdx.x");
        if (pencil)
        {
            for (long o = 0; o < O; ++o) out << "    double acc" << o << " = 0.0;\n";
            out << "    {\n        const long g = " << gExpr << ";\n";
            out << "#pragma unroll 1\n";
            out << "        for (long c = g * " << Sn << " + lane; c < " << Nc << "; c += " << G * Sn << ")\n        {\n";
            decompose(s.contr, "c", "            ");
            // operand bases (contraction part of the address) and memoised loads (output part is a literal)
            std::vector<std::string> loads, sums;
            std::map<std::string, std::string> memo;
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                const VarRef &r = s.in[v];
                std::string base = uvars[r.uvar].viewOffset != 0 ? Lit(uvars[r.uvar].viewOffset) : std::string();
                for (size_t d = 0; d < r.idx.size(); ++d)
                {
                    if (has(s.contr, r.idx[d])) base += (base.empty() ? "" : " + ") + IdxVar(r.idx[d]) + " * " + Lit(r.stride[d]);
                }
                out << "            const " << OffsetType() << " ob" << v << " = " << (base.empty() ? "0" : base) << ";\n";
            }
            std::vector<int> value(nidx, 0);
            for (long o = 0; o < O; ++o)
            {
                long rem = o;
                for (int j = static_cast<int>(s.outIdx.size()) - 1; j >= 0; --j)
                {
                    value[s.outIdx[j]] = static_cast<int>(rem % extent[s.outIdx[j]]);
                    rem /= extent[s.outIdx[j]];
                }
                std::string prod;
                for (size_t v = 0; v < s.in.size(); ++v)
                {
                    const VarRef &r = s.in[v];
                    long lit = 0;
                    for (size_t d = 0; d < r.idx.size(); ++d)
                    {
                        if (!has(s.contr, r.idx[d])) lit += static_cast<long>(value[r.idx[d]]) * r.stride[d];
                    }
                    const std::string key = str(static_cast<long>(v)) + ":" + str(lit);
                    auto it = memo.find(key);
                    if (it == memo.end())
                    {
                        const std::string name = "x" + str(static_cast<long>(v)) + "_" + str(static_cast<long>(memo.size()));
                        loads.push_back("const double " + name + " = " + PtrName(r.uvar) + "[ob" + str(static_cast<long>(v)) + " + " + Lit(lit) + "];");
                        it = memo.emplace(key, name).first;
                    }
                    prod = prod.empty() ? it->second : "(" + prod + " * " + it->second + ")";
                }
                sums.push_back("acc" + str(o) + " += " + prod + ";");
            }
            for (const auto &l : loads) out << "            " << l << "\n";
            for (const auto &l : sums) out << "            " << l << "\n";
            out << "        }\n    }\n";
            // lanes -> 64 lanes -> one: fixed order, whatever the timing
            for (long o = 0; o < O; ++o) out << "    red[lane * " << O << " + " << o << "] = acc" << o << ";\n";
            out << "    __syncthreads();\n";
            out << "    if (lane < 64)\n    {\n";
            out << "        for (int o = 0; o < " << O << "; ++o)\n        {\n            double t = 0.0;\n";
            out << "            for (int j = 0; j < " << NTr / 64 << "; ++j) t += red[(lane + 64 * j) * " << O << " + o];\n";
            out << "            red[lane * " << O << " + o] = t;\n        }\n    }\n";
            out << "    __syncthreads();\n";
            out << "    if (lane < " << O << ")\n    {\n        double t = 0.0;\n";
            out << "        for (int k = 0; k < 64; ++k) t += red[k * " << O << " + lane];\n";
        }
        else if (byRows)
        {
            out << "    const int og = blockIdx.x % " << Go << ", gc = blockIdx.x / " << Go << ";\n";
            out << "    const int o = og * " << Ow << " + lane / " << Sn << ", sl = lane % " << Sn << ";\n";
            out << "    double sum = 0.0;\n";
            out << "    if (o < " << O << ")\n    {\n";
            decompose(s.outIdx, "o", "        ");
            out << "#pragma unroll 4\n";   // (8: 77 -> 71 % of the HBM peak for 64 rows of 2^20 terms)
            out << "        for (long c = (long)gc * " << Sn << " + sl; c < " << Nc << "; c += " << G * Sn << ")\n        {\n";
            decompose(s.contr, "c", "            ");
            std::string prod;
            for (const auto &r : s.in)
            {
                const std::string opnd = PtrName(r.uvar) + "[" + FullOffset(r) + "]";
                prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
            }
            out << "            sum += " << prod << ";\n        }\n    }\n";
            out << "    red[lane] = sum;\n    __syncthreads();\n";
            // 16 lanes per output add four slices each, then one lane adds the 16: a fixed order
            out << "    if (lane < " << Ow * 16 << ")\n    {\n        double t = 0.0;\n";
            out << "        for (int k = 0; k < " << Sn / 16 << "; ++k) t += red[(lane / 16) * " << Sn << " + (lane % 16) * " << Sn / 16 << " + k];\n";
            out << "        red[" << NTr << " + lane] = t;\n    }\n    __syncthreads();\n";
            out << "    if (lane < " << Ow << " && og * " << Ow << " + lane < " << O << ")\n    {\n        double t = 0.0;\n";
            out << "        for (int k = 0; k < 16; ++k) t += red[" << NTr << " + lane * 16 + k];\n";
            out << "        scratch[(long)gc * " << O << " + og * " << Ow << " + lane] = t;\n    }\n}\n";
        }
        else
        {
            if (outputsFastest)
                out << "    const int sl = lane / " << O << ", o = lane % " << O << ";\n";
            else
                out << "    const int o = lane / " << Sn << ", sl = lane % " << Sn << ";\n";
            out << "    double sum = 0.0;\n";
            out << "    if (lane < " << Sn * O << ")\n    {\n";
            decompose(s.outIdx, "o", "        ");
            out << "        const long g = " << gExpr << ";\n";
            out << "#pragma unroll 8\n";   // (4: 71 %, 8: 75 %, 16: 74 % of the HBM peak for 64 column sums over 2^20 rows)
            out << "        for (long c = g * " << Sn << " + sl; c < " << Nc << "; c += " << G * Sn << ")\n        {\n";
            decompose(s.contr, "c", "            ");
            std::string prod;
            for (const auto &r : s.in)
            {
                const std::string opnd = PtrName(r.uvar) + "[" + FullOffset(r) + "]";
                prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
            }
            out << "            sum += " << prod << ";\n        }\n    }\n";
            out << "    red[lane] = sum;\n    __syncthreads();\n";
            out << "    if (lane < " << O << ")\n    {\n        double t = 0.0;\n";
            out << "        for (int k = 0; k < " << Sn << "; ++k) t += red["
                << (outputsFastest ? "k * " + str(O) + " + lane" : "lane * " + str(Sn) + " + k") << "];\n";
        }
        if (byRows)
        {
            // written above
        }
        else if (twoKernels)
            out << "        scratch[(long)blockIdx.x * " << O << " + lane] = t;\n    }\n}\n";
        else
            out << "        __hip_atomic_store(&scratch[(long)blockIdx.x * " << O
                << " + lane], t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n    }\n";

        // ---- stage 2: add the per-workgroup partials in a fixed order and apply the assignment operator.
        // Default: a second, single-workgroup kernel.
        // ACRO_HIP_ONE_PASS=1: the workgroup that arrives last at a device-wide counter does it instead (partials
        // written with device-scope atomic stores, arrival counted with a release, the last workgroup acquires; the
        // counter lives behind the partials in the scratch buffer, which the executor zeroes when it allocates it,
        // and the last workgroup sets it back to zero).  A release at device scope writes back the L2 of the
        // workgroup's XCD; with 256 workgroups the single launch measured 18.4 us against 16.3 us for the two
        // launches (55.9 us when every lane also fenced), so it is not the default.
        auto emitFinish = [&](const std::string &load) {
            out << "    const int g2 = lane / " << O << ", o2 = lane % " << O << ";\n";
            out << "    double sum2 = 0.0;\n";
            out << "    if (lane < " << S2 * O << ")\n    {\n";
            out << "#pragma unroll 8\n";
            out << "        for (long g = g2; g < " << G << "; g += " << S2 << ") sum2 += " << load << ";\n    }\n";
            out << "    red[lane] = sum2;\n    __syncthreads();\n";
            out << "    if (lane < " << O << ")\n    {\n        double t = 0.0;\n";
            out << "        for (int k = 0; k < " << S2 << "; ++k) t += red[k * " << O << " + lane];\n";
            decompose(s.outIdx, "lane", "        ");
            const std::string dst = (twoKernels ? std::string("result") : PtrName(s.out.uvar)) + "[" + FullOffset(s.out) + "]";
            if (s.op == '=')
                out << "        " << dst << " = t;\n";
            else
                out << "        " << dst << " = " << dst << (s.op == '+' ? " + t;\n" : " - t;\n");
            out << "    }\n";
        };
        if (twoKernels)
        {
            out << "\nextern \"C\" __global__ __launch_bounds__(" << NTf << ") void " << fFinal << "(double *"
                << (opt.noalias ? "__restrict__ " : "") << "result, const double *__restrict__ scratch)\n{\n";
            out << "    __shared__ double red[" << NTf << "];\n";
            out << "    const int lane = threadIdx.x;\n";
            emitFinish("scratch[g * " + str(O) + " + o2]");
            out << "}\n";
        }
        else
        {
            // The partials were stored by the wavefront of lane 0 with device-scope atomic stores; its release on the
            // counter orders them before the arrival.  Only the last workgroup needs the acquire side.
            // ACRO_HIP_ONE_PASS=2: the partials were written through to the device's point of coherence by the
            // atomic stores; the storing wavefront only waits until they are acknowledged (a workgroup-scope release)
            // and the arrival is counted without the device-scope release that writes back the XCD's L2.
            const bool light = envInt("ACRO_HIP_ONE_PASS") >= 2;
            if (light) out << "    __builtin_amdgcn_fence(__ATOMIC_RELEASE, \"workgroup\");\n";
            out << "    __syncthreads();\n";
            out << "    if (lane == 0)\n    {\n";
            out << "        const unsigned int arrived = __hip_atomic_fetch_add(" << counter
                << ", 1u, " << (light ? "__ATOMIC_RELAXED" : "__ATOMIC_RELEASE") << ", __HIP_MEMORY_SCOPE_AGENT);\n";
            out << "        isLast = (arrived == " << G - 1 << "u);\n    }\n";
            out << "    __syncthreads();\n";
            out << "    if (!isLast) return;\n";
            out << "    __threadfence();\n";
            emitFinish("__hip_atomic_load(&scratch[g * " + str(O) + " + o2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)");
            out << "    if (lane == 0) __hip_atomic_store(" << counter << ", 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
            out << "}\n";
        }

        plan.source = out.str();
        plan.scratch_doubles = static_cast<size_t>(G * O) + (twoKernels ? 0 : 1);
        plan.nb = 1;
        plan.lds_bytes = static_cast<int>((pencil ? NTr * O : NTr) * 8);
        FillParams(plan, false);
        const int S = static_cast<int>(stores.size());
        HipLaunch partial;
        partial.function_name = fPartial;
        partial.grid = static_cast<unsigned>(gridG);
        partial.block = NTr;
        for (int si = 0; si < S; ++si) partial.params.push_back(si);
        partial.params.push_back(-1);
        plan.launches.push_back(partial);
        if (twoKernels)
        {
            HipLaunch fin;
            fin.function_name = fFinal;
            fin.grid = 1;
            fin.block = NTf;
            fin.params.push_back(uvars[s.out.uvar].storage);
            fin.params.push_back(-1);
            plan.launches.push_back(fin);
        }
    }

    // ------------------------------------------------------------------------------ transpose schedule
    // A single kernel that only permutes the dimensions of one operand, with different, long fastest dimensions on
    // the two sides ("A_i_j = B_j_i" with 8 192 x 8 192 entries): whichever side the lanes follow, the other side
    // moves 8 bytes per 128-byte line (17 % of the HBM peak for that kernel).  Instead a workgroup moves a tile of
    // 32 x 32 entries through LDS: it reads rows of 32 consecutive entries along the operand's fastest dimension,
    // and writes rows of 32 consecutive entries along the output's.  The tile's rows are 33 doubles apart in LDS, so
    // that the transposed read is free of bank conflicts.
    bool UseTransposeSchedule() const
    {
        if (subs.size() != 1 || envInt("ACRO_HIP_TRANSPOSE") < 0 || !opt.noalias || NumGatherSlots() > 0) return false;
        const Sub &s = subs[0];
        if (s.matrixOp != 0 || s.in.size() != 1 || !s.contr.empty() || s.out.repeated || s.in[0].repeated) return false;
        if (s.in[0].uvar == s.out.uvar || s.in[0].idx.size() != s.out.idx.size() || s.out.idx.size() < 2) return false;
        const int a = s.in[0].idx.back(), b = s.out.idx.back();
        return a != b && extent[a] >= 32 && extent[b] >= 32;
    }

    void EmitTranspose(HipKernelPlan &plan)
    {
        const Sub &s = subs[0];
        const VarRef &in = s.in[0];
        const int a = in.idx.back(), b = s.out.idx.back();
        auto strideOf = [](const VarRef &r, int id) {
            for (size_t d = 0; d < r.idx.size(); ++d)
            {
                if (r.idx[d] == id) return r.stride[d];
            }
            return 0L;
        };
        std::vector<int> rest;
        for (int id : s.out.idx)
        {
            if (id != a && id != b) rest.push_back(id);
        }
        const long na = extent[a], nbb = extent[b], nrest = product(rest, extent);
        const int T = 32;  // entries per side of a tile (64 measured 55.4 against 58.7 % of the HBM peak for 8 192 x 8 192)
        const long tilesA = (na + T - 1) / T, tilesB = (nbb + T - 1) / T;
        const long groups = tilesA * tilesB * nrest;
        ACROBATIC_ASSERT(groups < (1L << 31), "HIP generator: too many tiles for one launch of the transpose schedule.");
        for (const auto &st : stores)
        {
            long entries = 1;
            for (int d : st.dims) entries *= d;
            if (entries >= (1L << 31) - 1) wide = true;
        }

        const std::string dimName = mk.GetDimensionedNameString();
        char hex[32];
        std::snprintf(hex, sizeof(hex), "%016llx",
                      static_cast<unsigned long long>(hashString(dimName + "/transpose/" + (Positional() ? "p" : "u"))));
        plan.module_name = std::string("acro_tr_") + hex;
        std::ostringstream sched;
        sched << "transpose schedule: tiles of " << T << " x " << T << " entries over (" << idxName[a] << ", " << idxName[b] << ") through LDS, "
              << groups << " workgroups of 256 lanes\n  [0] " << s.text << "\n";
        plan.schedule = sched.str();

        out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
        {
            std::istringstream lines(plan.schedule);
            std::string l;
            while (std::getline(lines, l)) out << "// " << l << "\n";
        }
        out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
        out << "    __shared__ double tile[" << T << " * " << T + 1 << "];\n";
        out << "    const int lx = threadIdx.x & " << T - 1 << ", ly = threadIdx.x / " << T << ";\n";
        out << "    long g = blockIdx.x;\n";
        // Tiles along a are taken in turn, and each starts at another tile along b: workgroups that run together then
        // write (and read) different column blocks.  With rows a power of two apart every tile of one column block
        // falls on the same memory channels (8 192 x 8 192: 57 % of the HBM peak in plain order, 65 % this way; the
        // diagonal along a instead, or shifted only every 8 tiles: 64 %, 60 %; tiles of 16 / 64 entries: 62 / 54 %).
        out << "    const int ta = (int)(g % " << tilesA << "); g /= " << tilesA << ";\n";
        out << "    const int tb = (int)((g % " << tilesB << " + ta) % " << tilesB << "); g /= " << tilesB << ";\n";
        std::string inBase = Lit(uvars[in.uvar].viewOffset), outBase = Lit(uvars[s.out.uvar].viewOffset);
        for (int j = static_cast<int>(rest.size()) - 1; j >= 0; --j)
        {
            const std::string name = IdxVar(rest[j]);
            out << "    const int " << name << " = (int)(g % " << extent[rest[j]] << "); g /= " << extent[rest[j]] << ";\n";
            inBase += " + " + name + " * " + Lit(strideOf(in, rest[j]));
            outBase += " + " + name + " * " + Lit(strideOf(s.out, rest[j]));
        }
        out << "    const " << OffsetType() << " inBase = " << inBase << ", outBase = " << outBase << ";\n";
        // the operand's rows run along a, the tile keeps them as rows
        out << "    for (int y = ly; y < " << T << "; y += " << 256 / T << ")\n    {\n";
        out << "        const int ia = ta * " << T << " + lx, ib = tb * " << T << " + y;\n";
        out << "        if (ia < " << na << " && ib < " << nbb << ") tile[y * " << T + 1 << " + lx] = " << PtrName(in.uvar) << "[inBase + ia * "
            << Lit(strideOf(in, a)) << " + ib * " << Lit(strideOf(in, b)) << "];\n    }\n";
        out << "    __syncthreads();\n";
        // the output's rows run along b: lane lx takes column lx of the tile's rows
        out << "    for (int y = ly; y < " << T << "; y += " << 256 / T << ")\n    {\n";
        out << "        const int ia = ta * " << T << " + y, ib = tb * " << T << " + lx;\n";
        out << "        if (ia < " << na << " && ib < " << nbb << ")\n        {\n";
        const std::string dst = PtrName(s.out.uvar) + "[outBase + ia * " + Lit(strideOf(s.out, a)) + " + ib * " + Lit(strideOf(s.out, b)) + "]";
        if (s.op == '=')
            out << "            " << dst << " = tile[lx * " << T + 1 << " + y];\n";
        else
            out << "            " << dst << " = " << dst << (s.op == '+' ? " + " : " - ") << "tile[lx * " << T + 1 << " + y];\n";
        out << "        }\n    }\n}\n";

        plan.source = out.str();
        plan.nb = 1;
        plan.lds_bytes = T * (T + 1) * 8;
        FillParams(plan, false);
        HipLaunch launch;
        launch.function_name = plan.module_name;
        launch.grid = static_cast<unsigned>(groups);
        launch.block = 256;
        for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
        plan.launches.push_back(launch);
    }

    // ------------------------------------------------------------------------------ operator schedule
    // One dense operator applied to every batch entry: "A_e_i = B_i_j X_e_j" with B too large for scalar operands or a
    // register tile (16 <= rows, columns; at most 4 096 entries), also with several row or column indices
    // ("A_e_i1_i2 = B_i1_i2_j1_j2 X_e_j1_j2") and with several leading indices numbering the entries
    // ("A_e_q_i = B_i_j X_e_q_j").  The generic schedule stages B in LDS and gives a lane one row and one
    // entry, which is bound by the 64 LDS reads per output (17 % of the HBM peak for 64 x 64).  Two variants:
    // rows a multiple of 16 and columns a multiple of 8 go to the FP64 matrix cores (EmitOperatorMatrixCores, 72 %;
    // the operator may then also be stored transposed, "B_j_i").  Otherwise a lane keeps its
    // row for four entries at a time, so one LDS read feeds four multiply-adds; the entry number is uniform in a
    // wavefront, so X is read with scalar loads, and the lanes of a wavefront write consecutive outputs (43 %).
    // Taking the entries' vectors into registers first and handing them round with readlane was slower (216 us).
    static constexpr int kOperatorEntriesPerLane = 4;

    // The kernels that the operator schedules see: the group's kernels, with pointwise kernels folded into the operator
    // kernel whose transient result they rescale ("U = B X" followed by "V = U D" reads as "V = B X D").
    mutable std::vector<Sub> opKernels;
    mutable bool opKernelsReady = false;

    void FoldPointwiseKernels() const
    {
        if (opKernelsReady) return;
        opKernelsReady = true;
        opKernels.clear();
        for (size_t k = 0; k < subs.size(); ++k)
        {
            const Sub &p = subs[k];
            bool folded = false;
            if (!opKernels.empty() && p.contr.empty() && p.op == '=' && p.matrixOp == 0 && !p.out.repeated && envInt("ACRO_HIP_OPERATOR_FOLD") >= 0)
            {
                Sub &m = opKernels.back();
                const int u = m.out.uvar;
                int reads = 0;
                bool sameShape = true;
                for (const auto &v : p.in)
                {
                    if (uvars[v.uvar].storage != uvars[u].storage) continue;
                    ++reads;
                    sameShape = sameShape && v.uvar == u && v.idx == m.out.idx && !v.repeated;
                }
                bool readLater = false;
                for (size_t j = k + 1; j < subs.size(); ++j)
                {
                    for (const auto &v : subs[j].in) readLater = readLater || uvars[v.uvar].storage == uvars[u].storage;
                    readLater = readLater || uvars[subs[j].out.uvar].storage == uvars[u].storage;
                }
                if (reads == 1 && sameShape && !readLater && m.op == '=' && !m.contr.empty() && p.out.idx == m.out.idx &&
                    stores[uvars[u].storage].transient && uvars[p.out.uvar].storage != uvars[u].storage)
                {
                    for (const auto &v : p.in)
                    {
                        if (v.uvar != u) m.in.push_back(v);
                    }
                    m.out = p.out;
                    m.text += " ; " + p.text;
                    folded = true;
                }
            }
            if (!folded) opKernels.push_back(p);
        }
    }
    int NumOpKernels() const
    {
        FoldPointwiseKernels();
        return static_cast<int>(opKernels.size());
    }
    const Sub &OpKernel(int k) const
    {
        FoldPointwiseKernels();
        return opKernels[k];
    }

    struct OperatorShape
    {
        const VarRef *op = nullptr, *x = nullptr;
        long rows = 0, cols = 0, entries = 0;
        bool transposed = false;   // the operator is stored with the contracted indices first: "B_j_i"
        bool cores = false;        // sizes and alignment suit the FP64 matrix cores
        bool pairs = false;        // the entries' vectors (and weights of their shape) come in 16-byte loads
        bool trailing = false;     // the entries are the fastest dimension: "A_i_e = B_i_j X_j_e"
        // > 1: the result and the vectors carry that many components behind the operator's indices
        // ("A_e_i_k = B_i_j X_e_j_k"): entry (e, k) has its vector elements and its outputs `comp` doubles apart
        long comp = 1;
        // Pointwise factors beside the operator and the vectors (matrix-core variant only): one value per entry
        // "W_e", per output "W_e_i", per row "W_i" scale the result; per vector element "W_e_j" or per column
        // "W_j" scale the entries' vectors as they are loaded.
        std::vector<const VarRef *> perEntry, perOutput, perRow, perElement, perColumn;
    };

    // `k`: the kernel of the group; `alone`: it is the whole group (inputs are then never written in the launch).
    bool OperatorPattern(OperatorShape &o, int k = 0, bool alone = true) const
    {
        if ((alone && NumOpKernels() != 1) || batch < 0 || !opt.noalias || NumGatherSlots() > 0 || envInt("ACRO_HIP_OPERATOR") < 0) return false;
        const Sub &s = OpKernel(k);
        if (s.matrixOp != 0 || s.in.size() < 2 || s.contr.empty() || s.out.repeated) return false;
        // the operator: the one operand without the batch index that carries contracted and free indices;
        // the vectors: the first operand with the batch index that carries every contracted index
        for (const auto &v : s.in)
        {
            bool contracted = false, free = false, all = true;
            for (int id : v.idx) (has(s.contr, id) ? contracted : free) = true;
            for (int id : s.contr) all = all && has(v.idx, id);
            if (!has(v.idx, batch) && contracted && free)
            {
                if (o.op) return false;
                o.op = &v;
            }
            else if (has(v.idx, batch) && all && !o.x)
                o.x = &v;
        }
        if (!o.op || !o.x) return false;
        for (const auto &v : s.in)
        {
            if (v.repeated || v.uvar == s.out.uvar || uvars[v.uvar].storage == uvars[s.out.uvar].storage) return false;
            if (alone && !IsPureInput(v.uvar)) return false;
        }
        // out = (e..., I...), X = (e..., J...), B = (I..., J...) or (J..., I...): the leading indices that the result
        // and X share, the batch index first, number the entries
        if (s.out.idx.empty()) return false;
        std::vector<int> lead, rows, cols;
        if (s.out.idx[0] == batch && o.x->idx[0] == batch)
        {
            size_t shared = 0;
            while (shared < s.out.idx.size() && shared < o.x->idx.size() && s.out.idx[shared] == o.x->idx[shared] &&
                   !has(o.op->idx, s.out.idx[shared]))
                ++shared;
            lead.assign(s.out.idx.begin(), s.out.idx.begin() + shared);
            rows.assign(s.out.idx.begin() + shared, s.out.idx.end());
            cols.assign(o.x->idx.begin() + shared, o.x->idx.end());
            // component indices: what the result and the vectors share behind the operator's indices
            while (rows.size() > 1 && cols.size() > 1 && rows.back() == cols.back() && !has(o.op->idx, rows.back()) &&
                   !has(s.contr, rows.back()))
            {
                o.comp *= extent[rows.back()];
                rows.pop_back();
                cols.pop_back();
            }
        }
        else
        {
            // or the trailing ones, the entries being the fastest dimension of the result and of X
            size_t shared = 0;
            const size_t no = s.out.idx.size(), nx = o.x->idx.size();
            while (shared < no && shared < nx && s.out.idx[no - 1 - shared] == o.x->idx[nx - 1 - shared] &&
                   !has(o.op->idx, s.out.idx[no - 1 - shared]))
                ++shared;
            lead.assign(s.out.idx.end() - shared, s.out.idx.end());
            rows.assign(s.out.idx.begin(), s.out.idx.end() - shared);
            cols.assign(o.x->idx.begin(), o.x->idx.end() - shared);
            o.trailing = true;
            if (!has(lead, batch)) return false;
        }
        if (rows.empty() || cols.empty()) return false;
        std::vector<int> plain = rows, swapped = cols;
        plain.insert(plain.end(), cols.begin(), cols.end());
        swapped.insert(swapped.end(), rows.begin(), rows.end());
        if (o.op->idx != plain && o.op->idx != swapped) return false;
        o.transposed = o.op->idx != plain;
        for (int id : cols)
        {
            if (!has(s.contr, id)) return false;
        }
        if (cols.size() != s.contr.size()) return false;
        o.rows = product(rows, extent);
        o.cols = product(cols, extent);
        o.entries = product(lead, extent) * o.comp;
        if (o.rows > 1024 || o.rows * o.cols > 4096) return false;
        // With components: vectors in 8-byte loads, no pointwise factors, and only where the generic schedule (an
        // entry and a row per lane) runs out of scalar registers for the operator or of coalescing for its stores
        // (64 x 64 with three components: 7 % of the HBM peak).
        if (o.comp > 1 && (s.in.size() != 2 || !alone || envInt("ACRO_HIP_OPERATOR_COMPONENTS") < 0)) return false;
        o.cores = envInt("ACRO_HIP_OPERATOR_MFMA") >= 0;
        // 16-byte loads: along the vectors, or along the entries where those are the fastest dimension
        o.pairs = (o.trailing ? o.entries % 2 == 0 && uvars[s.out.uvar].viewOffset % 2 == 0 : o.cols % 2 == 0) &&
                  uvars[o.x->uvar].viewOffset % 2 == 0 && o.comp == 1;
        for (const auto &v : s.in)
        {
            if (&v == o.op || &v == o.x) continue;
            const bool even = uvars[v.uvar].viewOffset % 2 == 0;
            if (v.idx == lead)
            {
                o.perEntry.push_back(&v);
                if (o.trailing) o.pairs = o.pairs && even;
            }
            else if (v.idx == s.out.idx)
            {
                o.perOutput.push_back(&v);
                if (o.trailing) o.pairs = o.pairs && even;
            }
            else if (v.idx == rows) o.perRow.push_back(&v);
            else if (v.idx == cols) o.perColumn.push_back(&v);
            else if (v.idx == o.x->idx)
            {
                o.perElement.push_back(&v);
                o.pairs = o.pairs && even;
            }
            else return false;
        }
        if (!o.cores) return o.rows >= 16 && o.cols >= 16 && !o.transposed && !o.trailing && s.in.size() == 2 && o.comp == 1;  // (its lanes walk the operator's rows)
        // A lane holds cols / 4 vector elements and rows / 4 results; the padded operator must fit the 64 KB of LDS
        // that a workgroup may declare.
        if (o.rows > 256 || o.cols > 256 || ((o.rows + 15) / 16 * 16) * ((o.cols + 7) / 8 * 8) > 8192) return false;
        if (o.trailing)
        {
            // Entries fastest: the generic schedule (one entry per lane, operator in scalar registers) streams whole
            // lines already; it falls behind as the operator grows (generic -> matrix cores: 8 x 8 86 -> 85 %,
            // 16 x 16 82 -> 84 %, 27 x 27 64 -> 78 %, 32 x 32 72 -> 80 %, 64 x 64 3 -> 65 %).  Two entries per lane
            // cost a large operator its registers (64 x 64: 72 us against 52 us with one entry per lane).
            if (o.rows * o.cols >= 2048) o.pairs = false;
            return o.rows * o.cols >= 512;
        }
        // Small operators: the generic schedule (operator in scalar registers, an entry or an output per lane) reads
        // and writes short pieces per lane and reaches 40 - 65 % of the HBM peak; 16 entries per wavefront on the
        // matrix cores reach 70 - 88 % as long as the entries' vectors come in 16-byte loads (even length) and five
        // or more rows fill the stores, or the vectors are long.  Measured wins: 8 x 4 53 -> 73 %, 16 x 4 43 -> 84 %,
        // 8 x 8 61 -> 85 %, 10 x 10 52 -> 81 %, 8 x 16 62 -> 85 %, 3 x 27 41 -> 73 %; losses, hence excluded:
        // 4 x 4 65 -> 49 %, 4 x 8 82 -> 77 %, 7 x 9 62 -> 57 %, 27 x 3 36 -> 28 %; 20 x 5 a tie.
        // (odd lengths: 9 x 9 47 -> 59 %, 25 x 25 45 -> 68 %, 27 x 27 46 -> 66 %; 5 x 5 63 -> 58 %)
        if (o.comp > 1) return o.rows * o.cols >= envInt("ACRO_HIP_OPERATOR_COMPONENTS_MIN", 256);
        return o.pairs ? (o.rows >= 5 && o.cols >= 4) : (o.cols >= 16 || (o.cols >= 9 && o.rows >= 8));
    }

    // A group of several kernels each of which is a large dense operator applied to every entry ("U = B X D" followed
    // by "Y = Bt U": a dense element operator applied and applied back) runs as one matrix-core launch per kernel,
    // in order on the stream, with the intermediates in device memory.  The fused chain schedule keeps the
    // intermediates on chip but gives a lane one entry and one row, which for large operators is bound by LDS reads:
    // 64 x 64, 2^18 entries: 400 us fused against 134 us for the two launches; 27 x 27: 241 against 143 us; small
    // operators stay fused (8 x 8 with a transient intermediate: 156 against 227 us; 12 x 10: 124 against 165 us).
    bool UseOperatorSequence() const
    {
        if (NumOpKernels() < 2 || envInt("ACRO_HIP_OPERATOR_SEQUENCE") < 0) return false;
        for (int k = 0; k < NumOpKernels(); ++k)
        {
            OperatorShape o;
            if (!OperatorPattern(o, k, false) || !o.cores || o.rows * o.cols < 512) return false;
        }
        return true;
    }

    // Two operator-shaped kernels of which the second is applied to the first one's result: one kernel, the
    // intermediate handed over through LDS (and stored as well unless it is transient).
    bool OperatorPair(OperatorShape &first, OperatorShape &second) const
    {
        if (NumOpKernels() != 2 || envInt("ACRO_HIP_OPERATOR_PAIR") < 0) return false;
        if (!OperatorPattern(first, 0, false) || !OperatorPattern(second, 1, false)) return false;
        if (!first.cores || !second.cores || first.trailing || second.trailing || first.comp > 1 || second.comp > 1) return false;
        const Sub &k0 = OpKernel(0), &k1 = OpKernel(1);
        if (k0.op != '=' || second.x->uvar != k0.out.uvar || second.x->idx != k0.out.idx) return false;
        if (uvars[k1.out.uvar].storage == uvars[k0.out.uvar].storage) return false;
        for (const auto &v : k1.in)
        {
            if (&v != second.x && uvars[v.uvar].storage == uvars[k0.out.uvar].storage) return false;
        }
        if (first.entries != second.entries || first.rows != second.cols) return false;
        // (2^19 - 2^22 entries, generic fused chain -> this kernel: 8 x 8 156 -> 142 us, 12 x 10 124 -> 93 us, 16 x 16 137 -> 61 us,
        // 20 x 12 125 -> 64 us, 24 x 20 277 -> 169 us; against two launches: 27 x 27 143 -> 74 us, 32 x 27 112 -> 62 us,
        // 64 x 27 190 -> 92 us)
        if (first.rows * first.cols < 64 || second.rows * second.cols < 64) return false;
        const long n1 = ((first.rows + 15) / 16 * 16) * (first.pairs ? (first.cols + 7) / 8 * 8 : (first.cols + 3) / 4 * 4);
        const long n2 = ((second.rows + 15) / 16 * 16) * ((second.cols + 3) / 4 * 4);
        return (n1 + n2 + 64 * (first.rows + 1)) * 8 <= 64 * 1024;
    }

    bool UseOperatorSchedule() const
    {
        OperatorShape o, o2;
        return OperatorPattern(o) || OperatorPair(o, o2) || UseOperatorSequence();
    }


    int opSub = 0;            // the kernel that the operator emitters work on
    bool opSequence = false;  // ... as one of several launches

    void EmitOperator(HipKernelPlan &plan)
    {
        {
            OperatorShape first, second;
            if (OperatorPair(first, second))
            {
                opSub = 0;
                EmitOperatorMatrixCores(plan, first, &second, 1);
                return;
            }
        }
        if (NumOpKernels() > 1)
        {
            opSequence = true;
            std::string schedule;
            int lds = 0;
            for (int k = 0; k < NumOpKernels(); ++k)
            {
                opSub = k;
                OperatorShape shape;
                OperatorPattern(shape, opSub, false);
                if (shape.trailing)
                    EmitOperatorEntriesFastest(plan, shape);
                else
                    EmitOperatorMatrixCores(plan, shape);
                schedule += plan.schedule;
                lds = std::max(lds, plan.lds_bytes);
            }
            plan.schedule = schedule;
            plan.lds_bytes = lds;
            plan.module_name = plan.launches.front().function_name;
            return;
        }
        const Sub &s = OpKernel(0);
        OperatorShape shape;
        OperatorPattern(shape);
        const VarRef *opr = shape.op, *x = shape.x;
        const long nJ = shape.cols, nI = shape.rows;
        const long E = shape.entries;        // entries of this schedule: all leading indices together
        if (shape.cores)
        {
            if (shape.trailing)
                EmitOperatorEntriesFastest(plan, shape);
            else
                EmitOperatorMatrixCores(plan, shape);
            return;
        }
        const int R = kOperatorEntriesPerLane;
        const long LI = (nI + 63) / 64 * 64;             // lanes per group of R entries: whole wavefronts
        // 512 lanes: the operator's copy in LDS allows four workgroups per CU, and the scalar loads of X come straight
        // from device memory, so the wavefronts in flight are what hides their latency (64 x 64: 104 us with 256
        // lanes, 87 us with 512, 93 us with 1 024).
        const int NTo = static_cast<int>(std::max<long>(512, LI));
        const long rowStride = nJ % 2 == 0 ? nJ + 1 : nJ;  // odd: the lanes' rows start in different LDS banks
        // Entries per workgroup: enough for the copy of B to stay small against what the entries move.
        // (64 x 64: 143 us with 16 entries per workgroup, 104 us with 64, the same with 128.)
        long groupsPerBlock = std::max<long>(1, (nI * nJ / 64 + R - 1) / R);
        groupsPerBlock = std::max<long>(groupsPerBlock, NTo / LI);
        const long NBo = groupsPerBlock * R;
        const long blocks = (E + NBo - 1) / NBo;
        for (const auto &st : stores)
        {
            long entries = 1;
            for (int d : st.dims) entries *= d;
            if (entries >= (1L << 31) - 1) wide = true;
        }

        const std::string dimName = mk.GetDimensionedNameString();
        char hex[32];
        std::snprintf(hex, sizeof(hex), "%016llx",
                      static_cast<unsigned long long>(hashString(dimName + "/operator/" + (Positional() ? "p" : "u"))));
        plan.module_name = std::string("acro_op_") + hex;
        std::ostringstream sched;
        sched << "operator schedule: " << nI << " x " << nJ << " operator in LDS (row stride " << rowStride << "), " << NBo
              << " entries per workgroup of " << NTo << " lanes, a lane keeps its row for " << R << " entries\n  [0] " << s.text << "\n";
        plan.schedule = sched.str();

        out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
        {
            std::istringstream lines(plan.schedule);
            std::string l;
            while (std::getline(lines, l)) out << "// " << l << "\n";
        }
        const std::string B = PtrName(opr->uvar), X = PtrName(x->uvar), A = PtrName(s.out.uvar);
        const char *assign = s.op == '=' ? " = " : (s.op == '+' ? " += " : " -= ");
        out << "typedef const __attribute__((address_space(4))) double *acro_scalar_ptr;\n";
        out << "\nextern \"C\" __global__ __launch_bounds__(" << NTo << ") void " << plan.module_name << "(" << ParamList() << ")\n{\n";
        out << "    __shared__ double rows[" << nI * rowStride << "];\n";
        out << "    const int tid = threadIdx.x;\n";
        out << "    for (int i = tid; i < " << nI * nJ << "; i += " << NTo << ") rows[(i / " << nJ << ") * " << rowStride << " + i % " << nJ
            << "] = " << B << "[" << Lit(uvars[opr->uvar].viewOffset) << " + i];\n";
        out << "    __syncthreads();\n";
        out << "    const long e0 = (long)blockIdx.x * " << NBo << ";\n";
        out << "    for (int w = tid; w < " << groupsPerBlock * LI << "; w += " << NTo << ")\n    {\n";
        out << "        const int g = __builtin_amdgcn_readfirstlane(w / " << LI << ");  // whole wavefronts share the entries\n";
        out << "        const int i = w - g * " << LI << ";\n";
        out << "        const long e = e0 + g * " << R << ";\n";
        out << "        if (i >= " << nI << " || e >= " << E << ") continue;\n";
        out << "        const double *row = rows + i * " << rowStride << ";\n";
        out << "        const acro_scalar_ptr x = (acro_scalar_ptr)(" << X << " + " << Lit(uvars[x->uvar].viewOffset) << " + e * " << nJ
            << ");  // uniform: scalar loads\n";
        out << "        double *a = " << A << " + " << Lit(uvars[s.out.uvar].viewOffset) << " + e * " << nI << " + i;\n";
        out << "        if (e + " << R << " <= " << E << ")\n        {\n";
        for (int r = 0; r < R; ++r) out << "            double s" << r << " = 0.0;\n";
        // Eight terms per trip: the entry's operand words of one trip arrive in one scalar load per entry, and two
        // trips' worth in flight hide the scalar cache's latency (measured: 119 / 87 / 79 / 78 us at 2 / 4 / 8 / 16).
        out << "#pragma unroll 8\n";
        out << "            for (int j = 0; j < " << nJ << "; ++j)\n            {\n                const double b = row[j];\n";
        for (int r = 0; r < R; ++r) out << "                s" << r << " += b * x[" << r * nJ << " + j];\n";
        out << "            }\n";
        for (int r = 0; r < R; ++r) out << "            a[" << r * nI << "]" << assign << "s" << r << ";\n";
        out << "        }\n        else\n        {\n";
        out << "            for (int r = 0; e + r < " << E << "; ++r)\n            {\n                double sum = 0.0;\n";
        out << "                for (int j = 0; j < " << nJ << "; ++j) sum += row[j] * x[r * " << nJ << " + j];\n";
        out << "                a[r * " << nI << "]" << assign << "sum;\n            }\n        }\n    }\n}\n";

        plan.source = out.str();
        plan.nb = static_cast<int>(NBo);
        plan.lds_bytes = static_cast<int>(nI * rowStride * 8);
        FillParams(plan, false);
        HipLaunch launch;
        launch.function_name = plan.module_name;
        launch.grid = static_cast<unsigned>(blocks);
        launch.block = static_cast<unsigned>(NTo);
        for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
        plan.launches.push_back(launch);
    }

    // The same on the FP64 matrix cores: a wavefront takes 16 entries at a time and forms their nI outputs with
    // v_mfma_f64_16x16x4 (16 entries x 16 outputs x 4 terms per instruction).  The entries' vectors are the
    // instruction's first operand, read with ordinary 16-byte vector loads (lane = entry + 16 * term group); the
    // operator sits in LDS in the order the second operand wants it, one conflict-free 8-byte read per lane and
    // instruction; a lane holds outputs (entry 4r + lane / 16, output lane % 16) in register r, so one store
    // instruction writes four runs of 128 bytes.  The order of the terms inside a step is free as long as both
    // operands agree: term group g of step s stands for j = 8 (s / 2) + 2 g + s % 2, which makes the entry's two
    // doubles of a 16-byte load the operands of two successive steps.  MI355X's vector and matrix FP64 peaks are the
    // same; what the matrix cores save is operand delivery: no scalar loads and 1/16 of the LDS reads.
    // 64 x 64 on 2^18 entries: 47 - 51 us against 79 us with scalar loads (512 workgroups; 58 us with 1 024, 76 us
    // with 2 048; loading the next 16 entries ahead of the arithmetic made no difference).
    // With `next` (and its kernel `nextSub`) the result of this operator never leaves the chip: it is scaled, written
    // to a per-wavefront piece of LDS in the result layout (entry 4r + lane / 16, output lane % 16), read back in the
    // operand layout (entry lane % 16, term group lane / 16) and multiplied by the second operator.
    void EmitOperatorMatrixCores(HipKernelPlan &plan, const OperatorShape &shape, const OperatorShape *next = nullptr, int nextSub = -1)
    {
        const Sub &s = OpKernel(opSub);
        const VarRef &opr = *shape.op, &x = *shape.x;
        const long nI = shape.rows, nJ = shape.cols, E = shape.entries;
        // Sizes that the instruction's 16 x 4 blocks do not divide: the operator's copy in LDS is padded with zero
        // rows and columns, the entries' vectors read as zero past their end, outputs past the last row are not
        // stored.  Pairs of doubles (16-byte loads) need an even row length and an even first element.
        const bool pairs = shape.pairs;
        // (Vectors of odd length come in 8-byte loads, 32-byte pieces per entry.  Reading the 16 vectors of a trip as
        // one contiguous range into a per-wavefront piece of LDS first measured slower: 17 x 17 70 -> 58 %,
        // 33 x 33 63 -> 41 %, 9 x 9 59 -> 39 %; only 27 x 27 gained, 66 -> 70 %.)
        const long nIp = (nI + 15) / 16 * 16, nJp = pairs ? (nJ + 7) / 8 * 8 : (nJ + 3) / 4 * 4;
        const long tilesN = nIp / 16, steps = nJp / 4;
        const long steps2 = (nI + 3) / 4;                 // the second operator contracts over this one's rows
        const long midStride = nI % 2 == 0 ? nI + 1 : nI; // odd: the lanes' rows of the hand-over buffer start in different banks
        const long tiles = (E + 15) / 16;
        const bool ragged = E % 16 != 0;
        // Equal work per CU matters more than the number of wavefronts: 256 CUs, one or two workgroups each.
        // With one or two loads per lane and trip a wavefront has little in flight, and twice the wavefronts help
        // once the tensors exceed the 256 MB of last-level cache (8 x 8 on 2^23 entries: 227 us with 512
        // workgroups, 185 us with 1 024, 216 us with 2 048; 64 x 64 on 2^18: 47 / 54 / 62 us).
        const long most = pairs && nJp <= 16 ? 1024 : 512;
        const long blocks = std::max<long>(1, std::min<long>(most, (tiles + 3) / 4));
        for (const auto &st : stores)
        {
            long entries = 1;
            for (int d : st.dims) entries *= d;
            if (entries >= (1L << 31) - 1) wide = true;
        }
        const std::string dimName = mk.GetDimensionedNameString();
        char hex[32];
        std::snprintf(hex, sizeof(hex), "%016llx",
                      static_cast<unsigned long long>(hashString(dimName + "/operator-mfma/" + str(opSub) + "/" + (Positional() ? "p" : "u") + (pairs ? "2" : "1") + (next ? "+" : "") + (shape.comp > 1 ? "c" + str(shape.comp) : ""))));
        plan.module_name = std::string("acro_op_") + hex;
        std::ostringstream sched;
        sched << "operator schedule on the FP64 matrix cores: " << nI << " x " << nJ << (shape.transposed ? " operator (stored transposed)" : " operator")
              << " in LDS in operand order";
        if (nIp != nI || nJp != nJ) sched << " (padded to " << nIp << " x " << nJp << ")";
        if (shape.comp > 1) sched << ", " << shape.comp << " components per vector element";
        sched << ", " << E << " entries, 16 per wavefront and trip, "
              << tilesN * steps << " v_mfma_f64_16x16x4 per trip, " << blocks << " workgroups of 256 lanes\n  [" << opSub << "] " << s.text << "\n";
        if (next)
            sched << "  [" << nextSub << "] " << OpKernel(nextSub).text << " : " << next->rows << " x " << next->cols << (next->transposed ? " operator (stored transposed)" : " operator")
                  << " applied to the first result on chip (handed over through " << 16 * midStride * 8 << " bytes of LDS per wavefront)\n";
        plan.schedule = sched.str();

        if (opSub == 0) out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
        {
            std::istringstream lines(plan.schedule);
            std::string l;
            while (std::getline(lines, l)) out << "// " << l << "\n";
        }
        const std::string B = PtrName(opr.uvar), X = PtrName(x.uvar), A = PtrName(s.out.uvar);
        const bool stream = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
        // term group g (lane / 16) of step s stands for this j
        const std::string termOf = pairs ? "8 * (step >> 1) + 2 * (l >> 4) + (step & 1)" : "4 * step + (l >> 4)";
        out << (opSub == 0 ? "" : "\n") << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
        // Two doubles moved by one 16-byte instruction.  The type only promises the 8-byte alignment that every
        // operand has (a caller's device buffer, a slice at an odd offset of it); the hardware takes such
        // addresses for accesses to device memory.
        out << "typedef double acro_pair __attribute__((ext_vector_type(2), aligned(8)));\n";
        out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
        out << "    __shared__ double frag[" << nIp * nJp << "];\n";
        out << "    for (int f = threadIdx.x; f < " << nIp * nJp << "; f += 256)\n    {\n";
        out << "        const int l = f & 63, step = (f >> 6) % " << steps << ", t = (f >> 6) / " << steps << ";\n";
        out << "        const int row = 16 * t + (l & 15), j = " << termOf << ";\n";
        const std::string element = B + "[" + Lit(uvars[opr.uvar].viewOffset) + (shape.transposed ? " + j * " + str(nI) + " + row]" : " + row * " + str(nJ) + " + j]");
        if (nIp != nI || nJp != nJ)
            out << "        frag[f] = row < " << nI << " && j < " << nJ << " ? " << element << " : 0.0;\n    }\n";
        else
            out << "        frag[f] = " << element << ";\n    }\n";
        if (next)
        {
            // the second operator: its columns are the first one's rows, terms in natural order
            const long rows2P = (next->rows + 15) / 16 * 16;
            out << "    __shared__ double frag2[" << rows2P * steps2 * 4 << "];\n";
            out << "    __shared__ double stage[" << 4 * 16 * midStride << "];\n";
            out << "    for (int f = threadIdx.x; f < " << rows2P * steps2 * 4 << "; f += 256)\n    {\n";
            out << "        const int l = f & 63, step = (f >> 6) % " << steps2 << ", t = (f >> 6) / " << steps2 << ";\n";
            out << "        const int row = 16 * t + (l & 15), j = 4 * step + (l >> 4);\n";
            out << "        frag2[f] = row < " << next->rows << " && j < " << nI << " ? " << PtrName(next->op->uvar) << "[" << Lit(uvars[next->op->uvar].viewOffset)
                << (next->transposed ? " + j * " + str(next->rows) + " + row]" : " + row * " + str(nI) + " + j]") << " : 0.0;\n    }\n";
        }
        out << "    __syncthreads();\n";
        out << "    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;\n";
        // (A contiguous range of trips per workgroup instead of this stride: the same or up to 8 % slower.)
        out << "    const long waves = (long)gridDim.x * 4;\n";
        out << "    for (long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6); tile < " << tiles << "; tile += waves)\n    {\n";
        if (ragged)
            out << "        const long ex = tile * 16 + c < " << E << " ? tile * 16 + c : " << E - 1 << ";  // past the end: any valid entry, never stored\n";
        else
            out << "        const long ex = tile * 16 + c;\n";
        if (pairs)
        {
            out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + ex * " << nJ << " + 2 * g;\n";
            out << "        double2 xv[" << nJp / 8 << "];\n";
            out << "#pragma unroll\n";
            out << "        for (int q = 0; q < " << nJp / 8 << "; ++q) xv[q] = ";
            if (nJp != nJ) out << "8 * q + 2 * g >= " << nJ << " ? double2{0.0, 0.0} : ";
            out << "[&] { const acro_pair t = *reinterpret_cast<const acro_pair *>(x + 8 * q); return double2{t.x, t.y}; }();\n";
            for (const VarRef *w : shape.perElement)
            {
                out << "#pragma unroll\n";
                out << "        for (int q = 0; q < " << nJp / 8 << "; ++q)\n        {\n";
                if (nJp != nJ) out << "            if (8 * q + 2 * g >= " << nJ << ") continue;\n";
                out << "            const acro_pair f = *reinterpret_cast<const acro_pair *>(" << PtrName(w->uvar) << " + " << Lit(uvars[w->uvar].viewOffset)
                    << " + ex * " << nJ << " + 2 * g + 8 * q);\n            xv[q].x *= f.x;\n            xv[q].y *= f.y;\n        }\n";
            }
            for (const VarRef *w : shape.perColumn)
            {
                out << "#pragma unroll\n";
                out << "        for (int q = 0; q < " << nJp / 8 << "; ++q)\n        {\n";
                if (nJp != nJ) out << "            if (8 * q + 2 * g >= " << nJ << ") continue;\n";
                out << "            const double *f = " << PtrName(w->uvar) << " + " << Lit(uvars[w->uvar].viewOffset)
                    << " + 2 * g + 8 * q;\n            xv[q].x *= f[0];\n            xv[q].y *= f[1];\n        }\n";
            }
        }
        else
        {
            const long C = shape.comp;
            if (C > 1)
                out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + (ex / " << C << ") * " << nJ * C
                    << " + ex % " << C << " + g * " << C << ";\n";
            else
                out << "        const double *x = " << X << " + " << Lit(uvars[x.uvar].viewOffset) << " + ex * " << nJ << " + g;\n";
            out << "        double xv[" << steps << "];\n";
            out << "#pragma unroll\n";
            out << "        for (int q = 0; q < " << steps << "; ++q) xv[q] = ";
            if (nJp != nJ) out << "4 * q + g >= " << nJ << " ? 0.0 : ";
            out << "x[" << 4 * C << " * q];\n";
            for (const VarRef *w : shape.perElement)
            {
                out << "#pragma unroll\n";
                out << "        for (int q = 0; q < " << steps << "; ++q) ";
                if (nJp != nJ) out << "if (4 * q + g < " << nJ << ") ";
                out << "xv[q] *= " << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + ex * " << nJ << " + g + 4 * q];\n";
            }
            for (const VarRef *w : shape.perColumn)
            {
                out << "#pragma unroll\n";
                out << "        for (int q = 0; q < " << steps << "; ++q) ";
                if (nJp != nJ) out << "if (4 * q + g < " << nJ << ") ";
                out << "xv[q] *= " << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + g + 4 * q];\n";
            }
        }
        out << "        acro_double4 acc[" << tilesN << "];\n";
        out << "#pragma unroll\n";
        out << "        for (int t = 0; t < " << tilesN << "; ++t) acc[t] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
        out << "#pragma unroll\n";
        out << "        for (int step = 0; step < " << steps << "; ++step)\n        {\n";
        if (pairs)
            out << "            const double xs = (step & 1) ? xv[step >> 1].y : xv[step >> 1].x;\n";
        else
            out << "            const double xs = xv[step];\n";
        out << "#pragma unroll\n";
        out << "            for (int t = 0; t < " << tilesN << "; ++t)\n";
        out << "                acc[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(xs, frag[(t * " << steps << " + step) * 64 + lane], acc[t], 0, 0, 0);\n";
        out << "        }\n";
        // Stores of one operator's results (or, with toLds, their hand-over to the second operator).
        auto emitResults = [&](const Sub &ks, const OperatorShape &sh, long rows, const std::string &accName, bool toLds) {
            const long rowsP = (rows + 15) / 16 * 16;
            const bool streams = ks.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
            const long C = sh.comp;
            if (!toLds && C == 1)
                out << "        double *a = " << PtrName(ks.out.uvar) << " + " << Lit(uvars[ks.out.uvar].viewOffset) << " + (tile * 16 + g) * " << rows << " + c;\n";
            out << "#pragma unroll\n";
            out << "        for (int r = 0; r < 4; ++r)\n        {\n";
            if (ragged) out << "            if (tile * 16 + g + 4 * r >= " << E << ") continue;\n";
            if (!toLds && C > 1)
            {
                // entry (e, k): its outputs lie C doubles apart
                out << "            const long en_ = tile * 16 + g + 4 * r;\n";
                out << "            double *a = " << PtrName(ks.out.uvar) << " + " << Lit(uvars[ks.out.uvar].viewOffset) << " + (en_ / " << C << ") * "
                    << rows * C << " + en_ % " << C << " + c * " << C << ";\n";
            }
            // the result's pointwise factors
            std::string value = accName + "[t][r]";
            const bool scaled = !sh.perEntry.empty() || !sh.perOutput.empty() || !sh.perRow.empty();
            if (scaled) out << "            const long en = tile * 16 + g + 4 * r;\n";
            if (!sh.perEntry.empty())
            {
                out << "            const double se = ";
                for (size_t i = 0; i < sh.perEntry.size(); ++i)
                    out << (i ? " * " : "") << PtrName(sh.perEntry[i]->uvar) << "[" << Lit(uvars[sh.perEntry[i]->uvar].viewOffset) << " + en]";
                out << ";\n";
                value += " * se";
            }
            for (const VarRef *w : sh.perOutput)
                value += " * " + PtrName(w->uvar) + "[" + Lit(uvars[w->uvar].viewOffset) + " + en * " + str(rows) + " + 16 * t + c]";
            for (const VarRef *w : sh.perRow)
                value += " * " + PtrName(w->uvar) + "[" + Lit(uvars[w->uvar].viewOffset) + " + 16 * t + c]";
            out << "#pragma unroll\n";
            out << "            for (int t = 0; t < " << rowsP / 16 << "; ++t)\n";
            std::string guard = rowsP != rows ? "if (16 * t + c < " + str(rows) + ") " : "";
            if (toLds)
                out << "                " << guard << "mid[(4 * r + g) * " << midStride << " + 16 * t + c] = " << value << ";\n";
            else if (C > 1)
                out << "                " << guard << "a[" << 16 * C << " * t]" << (ks.op == '=' ? " = " : (ks.op == '+' ? " += " : " -= ")) << value << ";\n";
            else if (streams)
                out << "                " << guard << "__builtin_nontemporal_store(" << value << ", a + 4 * r * " << rows << " + 16 * t);\n";
            else
                out << "                " << guard << "a[4 * r * " << rows << " + 16 * t]" << (ks.op == '=' ? " = " : (ks.op == '+' ? " += " : " -= ")) << value << ";\n";
            out << "        }\n";
        };
        (void)A;
        (void)stream;
        if (!next)
            emitResults(s, shape, nI, "acc", false);
        else
        {
            const long rows2 = next->rows, rows2P = (rows2 + 15) / 16 * 16;
            out << "        double *mid = stage + (threadIdx.x >> 6) * " << 16 * midStride << ";\n";
            out << "        {\n";
            emitResults(s, shape, nI, "acc", true);
            out << "        }\n";
            if (!stores[uvars[s.out.uvar].storage].transient)
            {
                // the first result is wanted in device memory as well
                out << "        {\n";
                emitResults(s, shape, nI, "acc", false);
                out << "        }\n";
            }
            // a wavefront's LDS accesses complete in program order: no barrier, only the compiler kept from reordering
            out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
            out << "        acro_double4 acc2[" << rows2P / 16 << "];\n";
            out << "#pragma unroll\n";
            out << "        for (int t = 0; t < " << rows2P / 16 << "; ++t) acc2[t] = acro_double4{0.0, 0.0, 0.0, 0.0};\n";
            out << "#pragma unroll\n";
            out << "        for (int step = 0; step < " << steps2 << "; ++step)\n        {\n";
            out << "            const double us = ";
            if (steps2 * 4 != nI) out << "4 * step + g >= " << nI << " ? 0.0 : ";
            out << "mid[c * " << midStride << " + 4 * step + g]";
            // the second kernel's factors on its operand side: per element of the intermediate, or per column
            const std::string inRange = steps2 * 4 != nI ? "(4 * step + g < " + str(nI) + " ? " : "";
            const std::string otherwise = steps2 * 4 != nI ? " : 0.0)" : "";
            for (const VarRef *w : next->perElement)
                out << " * " << inRange << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + ex * " << nI << " + 4 * step + g]" << otherwise;
            for (const VarRef *w : next->perColumn)
                out << " * " << inRange << PtrName(w->uvar) << "[" << Lit(uvars[w->uvar].viewOffset) << " + 4 * step + g]" << otherwise;
            out << ";\n";
            out << "#pragma unroll\n";
            out << "            for (int t = 0; t < " << rows2P / 16 << "; ++t)\n";
            out << "                acc2[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(us, frag2[(t * " << steps2 << " + step) * 64 + lane], acc2[t], 0, 0, 0);\n";
            out << "        }\n";
            out << "        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, \"wavefront\");\n        __builtin_amdgcn_wave_barrier();\n";
            emitResults(OpKernel(nextSub), *next, rows2, "acc2", false);
        }
        out << "    }\n}\n";


        plan.source = out.str();
        plan.nb = 64;
        plan.lds_bytes = static_cast<int>((nIp * nJp + (next ? (next->rows + 15) / 16 * 16 * steps2 * 4 + 64 * midStride : 0)) * 8);
        FillParams(plan, false);
        HipLaunch launch;
        launch.function_name = plan.module_name;
        launch.grid = static_cast<unsigned>(blocks);
        launch.block = 256;
        for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
        plan.launches.push_back(launch);
    }

    // The same with the entries as the fastest dimension ("A_i_e = B_i_j X_j_e"): the roles of the instruction's operands
    // are exchanged.  The operator is the first operand (16 rows x 4 terms per instruction, from LDS in operand order),
    // the entries' vectors the second: lane = entry + 16 * term group reads X[j][e], 16 consecutive entries per term, and
    // result register r of a lane holds row 4r + lane / 16 of its entry, so loads and stores run along the entries.
    // With an even number of entries a wavefront takes 32 entries per trip: a lane loads two neighbouring entries in
    // 16 bytes, which feed two accumulator sets (even and odd entries), and stores its two results together.
    void EmitOperatorEntriesFastest(HipKernelPlan &plan, const OperatorShape &shape)
    {
        const Sub &s = OpKernel(opSub);
        const VarRef &opr = *shape.op, &x = *shape.x;
        const long nI = shape.rows, nJ = shape.cols, E = shape.entries;
        const bool pairs = shape.pairs;
        const int per = pairs ? 32 : 16;
        const long nIp = (nI + 15) / 16 * 16, nJp = (nJ + 3) / 4 * 4;
        const long tilesM = nIp / 16, steps = nJp / 4;
        const long trips = (E + per - 1) / per;
        const bool ragged = E % per != 0;
        const long blocks = std::max<long>(1, std::min<long>(512, (trips + 3) / 4));
        for (const auto &st : stores)
        {
            long entries = 1;
            for (int d : st.dims) entries *= d;
            if (entries >= (1L << 31) - 1) wide = true;
        }
        const std::string dimName = mk.GetDimensionedNameString();
        char hex[32];
        std::snprintf(hex, sizeof(hex), "%016llx",
                      static_cast<unsigned long long>(hashString(dimName + "/operator-mfma-t/" + str(opSub) + "/" + (Positional() ? "p" : "u") + (pairs ? "2" : "1"))));
        plan.module_name = std::string("acro_op_") + hex;
        std::ostringstream sched;
        sched << "operator schedule on the FP64 matrix cores, entries fastest: " << nI << " x " << nJ
              << (shape.transposed ? " operator (stored transposed)" : " operator") << " in LDS in operand order";
        if (nIp != nI || nJp != nJ) sched << " (padded to " << nIp << " x " << nJp << ")";
        sched << ", " << E << " entries, " << per << " per wavefront and trip, " << tilesM * steps * (pairs ? 2 : 1)
              << " v_mfma_f64_16x16x4 per trip, " << blocks << " workgroups of 256 lanes\n  [" << opSub << "] " << s.text << "\n";
        plan.schedule = sched.str();

        if (opSub == 0) out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
        {
            std::istringstream lines(plan.schedule);
            std::string l;
            while (std::getline(lines, l)) out << "// " << l << "\n";
        }
        const std::string B = PtrName(opr.uvar), X = PtrName(x.uvar), A = PtrName(s.out.uvar);
        const bool stream = s.op == '=' && envInt("ACRO_HIP_NT_STORE") >= 0;
        const std::string vt = pairs ? "acro_double2" : "double";
        auto offsetOf = [&](const VarRef &v) { return Lit(uvars[v.uvar].viewOffset); };
        out << (opSub == 0 ? "" : "\n") << "typedef double acro_double4 __attribute__((ext_vector_type(4)));\n";
        // only the 8-byte alignment that every operand has is promised (see acro_pair in the other operator kernel)
        out << "typedef double acro_double2 __attribute__((ext_vector_type(2), aligned(8)));\n";
        out << "\nextern \"C\" __global__ __launch_bounds__(256) void " << plan.module_name << "(" << ParamList() << ")\n{\n";
        out << "    __shared__ double frag[" << nIp * nJp << "];\n";
        out << "    for (int f = threadIdx.x; f < " << nIp * nJp << "; f += 256)\n    {\n";
        out << "        const int l = f & 63, step = (f >> 6) % " << steps << ", t = (f >> 6) / " << steps << ";\n";
        out << "        const int row = 16 * t + (l & 15), j = 4 * step + (l >> 4);\n";
        const std::string element = B + "[" + offsetOf(opr) + (shape.transposed ? " + j * " + str(nI) + " + row]" : " + row * " + str(nJ) + " + j]");
        if (nIp != nI || nJp != nJ)
            out << "        frag[f] = row < " << nI << " && j < " << nJ << " ? " << element << " : 0.0;\n    }\n";
        else
            out << "        frag[f] = " << element << ";\n    }\n";
        out << "    __syncthreads();\n";
        out << "    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;\n";
        out << "    const long waves = (long)gridDim.x * 4;\n";
        out << "    for (long trip = (long)blockIdx.x * 4 + (threadIdx.x >> 6); trip < " << trips << "; trip += waves)\n    {\n";
        out << "        const long e = trip * " << per << " + " << (pairs ? "2 * c" : "c") << ";\n";
        if (ragged)
            out << "        const long ex = e < " << E << " ? e : " << E - (pairs ? 2 : 1) << ";  // past the end: any valid entry, never stored\n";
        else
            out << "        const long ex = e;\n";
        out << "        " << vt << " xv[" << steps << "];\n";
        out << "#pragma unroll\n";
        out << "        for (int step = 0; step < " << steps << "; ++step)\n        {\n";
        out << "            const int j = 4 * step + g;\n";
        if (nJp != nJ) out << "            if (j >= " << nJ << ") { xv[step] = " << (pairs ? "acro_double2{0.0, 0.0}" : "0.0") << "; continue; }\n";
        out << "            xv[step] = *reinterpret_cast<const " << vt << " *>(" << X << " + " << offsetOf(x) << " + j * " << E << " + ex);\n";
        for (const VarRef *w : shape.perElement)
            out << "            xv[step] *= *reinterpret_cast<const " << vt << " *>(" << PtrName(w->uvar) << " + " << offsetOf(*w) << " + j * " << E << " + ex);\n";
        for (const VarRef *w : shape.perColumn)
            out << "            xv[step] *= " << PtrName(w->uvar) << "[" << offsetOf(*w) << " + j];\n";
        out << "        }\n";
        out << "        acro_double4 acc0[" << tilesM << "]" << (pairs ? ", acc1[" + str(tilesM) + "]" : "") << ";\n";
        out << "#pragma unroll\n";
        out << "        for (int t = 0; t < " << tilesM << "; ++t) acc0[t] = " << (pairs ? "acc1[t] = " : "") << "acro_double4{0.0, 0.0, 0.0, 0.0};\n";
        out << "#pragma unroll\n";
        out << "        for (int step = 0; step < " << steps << "; ++step)\n        {\n";
        out << "#pragma unroll\n";
        out << "            for (int t = 0; t < " << tilesM << "; ++t)\n            {\n";
        out << "                const double b = frag[(t * " << steps << " + step) * 64 + lane];\n";
        if (pairs)
        {
            out << "                acc0[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step].x, acc0[t], 0, 0, 0);\n";
            out << "                acc1[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step].y, acc1[t], 0, 0, 0);\n";
        }
        else
            out << "                acc0[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(b, xv[step], acc0[t], 0, 0, 0);\n";
        out << "            }\n        }\n";
        if (ragged) out << "        if (e >= " << E << ") continue;\n";
        if (!shape.perEntry.empty())
        {
            out << "        const " << vt << " se = ";
            for (size_t i = 0; i < shape.perEntry.size(); ++i)
                out << (i ? " * " : "") << "*reinterpret_cast<const " << vt << " *>(" << PtrName(shape.perEntry[i]->uvar) << " + " << offsetOf(*shape.perEntry[i]) << " + e)";
            out << ";\n";
        }
        out << "#pragma unroll\n";
        out << "        for (int t = 0; t < " << tilesM << "; ++t)\n";
        out << "#pragma unroll\n";
        out << "            for (int r = 0; r < 4; ++r)\n            {\n";
        out << "                const int i = 16 * t + 4 * r + g;\n";
        if (nIp != nI) out << "                if (i >= " << nI << ") continue;\n";
        out << "                " << vt << " v = " << (pairs ? "acro_double2{acc0[t][r], acc1[t][r]}" : "acc0[t][r]") << ";\n";
        if (!shape.perEntry.empty()) out << "                v *= se;\n";
        for (const VarRef *w : shape.perOutput)
            out << "                v *= *reinterpret_cast<const " << vt << " *>(" << PtrName(w->uvar) << " + " << offsetOf(*w) << " + i * " << E << " + e);\n";
        for (const VarRef *w : shape.perRow)
            out << "                v *= " << PtrName(w->uvar) << "[" << offsetOf(*w) << " + i];\n";
        out << "                " << vt << " *a = reinterpret_cast<" << vt << " *>(" << A << " + " << offsetOf(s.out) << " + i * " << E << " + e);\n";
        if (stream)
            out << "                __builtin_nontemporal_store(v, a);\n";
        else
            out << "                *a " << (s.op == '=' ? "= " : (s.op == '+' ? "+= " : "-= ")) << "v;\n";
        out << "            }\n    }\n}\n";

        plan.source = out.str();
        plan.nb = 64;
        plan.lds_bytes = static_cast<int>(nIp * nJp * 8);
        FillParams(plan, false);
        HipLaunch launch;
        launch.function_name = plan.module_name;
        launch.grid = static_cast<unsigned>(blocks);
        launch.block = 256;
        for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
        plan.launches.push_back(launch);
    }

    void Emit(HipKernelPlan &plan)
    {
        const int K = static_cast<int>(subs.size());
        const int U = static_cast<int>(uvars.size());
        const std::string dimName = mk.GetDimensionedNameString();
        std::string variant = str(NB) + "/" + str(NT) + "/" + (opt.noalias ? "n" : "a") + (Positional() ? "p" : "u") +
                              "/" + str(envInt("ACRO_HIP_PERSIST")) + (envInt("ACRO_HIP_PIPELINE") > 0 ? "p" + str(envInt("ACRO_HIP_PIPELINE")) : "") +
                              (envInt("ACRO_HIP_WAVES_PER_EU") > 0 ? "w" + str(envInt("ACRO_HIP_WAVES_PER_EU")) : "");
        for (const auto &st : stores) variant += st.elide ? "e" : (st.inLds ? "l" : "g");
        for (int u = 0; u < U; ++u) variant += "s" + str(uvars[u].storage) + "@" + str(uvars[u].viewOffset);
        for (int g : opt.gathered) variant += "g" + str(g);
        char hex[32];
        std::snprintf(hex, sizeof(hex), "%016llx", static_cast<unsigned long long>(hashString(dimName + variant)));
        plan.module_name = std::string("acro_mk_") + hex;
        const std::string function_name = plan.module_name;

        std::ostringstream sched;
        sched << "batch index " << (batch >= 0 ? idxName[batch] : std::string("(none)")) << " extent " << E << ", " << NB
              << " per workgroup of " << NT << " lanes, LDS " << ldsDoubles * 8 << " bytes\n";
        for (int k = 0; k < K; ++k)
        {
            const Sub &s = subs[k];
            sched << "  [" << k << "] " << s.text << " : lanes(";
            for (size_t j = 0; j < s.lane.size(); ++j) sched << (j ? "," : "") << idxName[s.lane[j]];
            sched << ")=" << s.laneCount << " tile(";
            for (size_t j = 0; j < s.tile.size(); ++j) sched << (j ? "," : "") << idxName[s.tile[j]];
            sched << ")=" << s.tileCount << " contraction=" << s.contrCount << (s.loopMode ? " looped" : " unrolled")
                  << (s.fusedWithPrev ? " in-register after previous" : "") << " phase " << s.phase << "; operands:";
            for (size_t v = 0; v < s.in.size(); ++v)
            {
                static const char *const names[] = {"registers", "scalar", "lds", "global"};
                const Source src = SourceOf(k, static_cast<int>(v));
                sched << " " << uvars[s.in[v].uvar].name << "<-"
                      << (src == kFromGlobal && GatherSlot(s.in[v].uvar) >= 0 ? "gathered" : names[src]);
            }
            const UVarInfo &uo = uvars[s.out.uvar];
            const bool elided = !StoresToGlobal(k);
            sched << "; " << uo.name << "->" << (NeedsLdsCopy(k) ? "lds" : "")
                  << (elided ? "" : (NeedsLdsCopy(k) ? "+global" : "global")) << "\n";
        }
        plan.schedule = sched.str();

        out << "// Generated by the acrotensor HIP code generator for gfx950.\n";
        {
            std::istringstream lines(plan.schedule);
            std::string l;
            while (std::getline(lines, l)) out << "// " << l << "\n";
        }
        out << "typedef const __attribute__((address_space(4))) double *acro_scalar_ptr;\n\n";
        out << "extern \"C\" __global__ __launch_bounds__(" << NT << ") ";
        // experiment switch: ask the compiler for a register budget that lets this many wavefronts share a SIMD
        if (envInt("ACRO_HIP_WAVES_PER_EU") > 0)
            out << "__attribute__((amdgpu_waves_per_eu(" << envInt("ACRO_HIP_WAVES_PER_EU") << ", " << envInt("ACRO_HIP_WAVES_PER_EU") << "))) ";
        out << "void " << function_name << "(";
        out << ParamList();
        out << ")\n{\n";
        if (ldsDoubles > 0) out << "    __shared__ double lds[" << ldsDoubles << "];\n";
        std::set<int> scalarStores;
        for (int k = 0; k < K; ++k)
        {
            for (size_t v = 0; v < subs[k].in.size(); ++v)
            {
                if (SourceOf(k, static_cast<int>(v)) == kFromConstant)
                    scalarStores.insert(uvars[subs[k].in[v].uvar].storage);
            }
        }
        for (int si : scalarStores)
            out << "    const acro_scalar_ptr C" << si << " = (acro_scalar_ptr)T" << si << ";\n";
        out << "    const int tid = threadIdx.x;\n";
        // Persistent form (ACRO_HIP_PERSIST=<workgroups per CU>): a fixed grid walks over the batch in a loop.
        const long totalGroups = (E + NB - 1) / NB;
        const long persist = envInt("ACRO_HIP_PERSIST");
        const long gridGroups = persist > 0 ? std::min<long>(totalGroups, persist * 256) : totalGroups;
        const bool looped = gridGroups < totalGroups;
        // Pipelined form of the persistent loop (ACRO_HIP_PIPELINE=1): the streaming inputs of every phase, the first
        // included, live in registers across iterations; a phase that has consumed its registers at once requests
        // the next batch entries' values, so that a workgroup never waits for device memory at the top of an
        // iteration and the memory system always holds requests of every resident workgroup.
        const bool pipelined = looped && envInt("ACRO_HIP_PIPELINE") > 0;
        const std::string loopHeader = "    for (int e0 = blockIdx.x * " + str(NB) + "; e0 < " + str(E) + "; e0 += " +
                                       str(gridGroups * NB) + ")\n    {\n";
        if (looped && !pipelined)
            out << loopHeader;
        else if (!looped)
            out << "    const int e0 = blockIdx.x * " << NB << ";\n    {\n";

        const bool guardBatch = (E % NB) != 0;

        bool anyStaged = false;
        for (size_t si = 0; si < stores.size(); ++si)
        {
            const Storage &st = stores[si];
            if (!st.staged || !st.inLds) continue;
            anyStaged = true;
            const UVarInfo &u = uvars[st.members[0]];
            out << "    {   // " << u.name << ": device memory -> LDS, once per workgroup\n";
            out << "        for (int i = tid; i < " << u.size << "; i += " << NT << ")\n        {\n";
            out << "            int r_ = i, a = " << st.ldsOffset << ";\n";
            long natural = u.size;
            for (size_t d = 0; d < st.dims.size(); ++d)
            {
                natural /= st.dims[d];
                if (d + 1 < st.dims.size())
                    out << "            a += (r_ / " << natural << ") * " << st.ldsStride[d] << "; r_ %= " << natural << ";\n";
                else
                    out << "            a += r_ * " << st.ldsStride[d] << ";\n";
            }
            out << "            lds[a] = T" << si << "[" << Lit(u.viewOffset) << " + i];\n        }\n    }\n";
        }
        if (anyStaged) out << "    __syncthreads();\n";

        // Work-item header: batch entry and lane indices of item `w` of the phase that kernel `ks` opens.
        auto emitHeader = [&](const Sub &s, const std::string &indent) {
            // A wavefront whose 64 items belong to one batch entry: say so, and the compiler turns loads that depend
            // on the entry alone into scalar loads.
            if (s.laneCount % 64 == 0 && envInt("ACRO_HIP_WAVE_UNIFORM") >= 0)
                out << indent << "const int b = __builtin_amdgcn_readfirstlane(w / " << s.laneCount << ");\n";
            else
                out << indent << "const int b = w / " << s.laneCount << ";\n";
            out << indent << "const int e = e0 + b;\n";
            if (!s.lane.empty())
            {
                out << indent << "const int r_ = w - b * " << s.laneCount << ";\n";
                long st = s.laneCount;
                for (size_t j = 0; j < s.lane.size(); ++j)
                {
                    const int id = s.lane[j];
                    st /= extent[id];
                    out << indent << "const int " << IdxVar(id) << " = ";
                    if (j == 0)
                        out << "r_ / " << st << ";\n";
                    else
                        out << "(r_ / " << st << ") % " << extent[id] << ";\n";
                }
            }
        };

        // Phases, the chains (a kernel plus the kernels applied in its registers) each of them runs side by side, and
        // what each may prefetch at kernel entry: the loads of streaming inputs of every phase after the first are
        // issued before the first phase starts, so that their latency overlaps with the earlier phases instead of
        // stalling a workgroup that few others can cover for.
        struct Chain
        {
            int first, last;
            long W;       // work items
            long offset;  // first item slot in the phase (multiple of the wavefront size)
            std::vector<std::vector<std::pair<std::string, std::string>>> loads;  // per kernel: prefetchable loads
            // per kernel and pass: memo key -> register name
            std::vector<std::vector<std::map<std::string, std::string>>> names;
        };
        struct Phase
        {
            std::vector<Chain> chains;
            long slots = 0, passes = 1;
            bool prefetched = false;
            bool carried = false;  // pipelined loop: the prefetched values are requested one iteration ahead
        };
        std::vector<Phase> phases;
        for (int k = 0; k < K;)
        {
            Chain c;
            c.first = k;
            c.last = k;
            while (c.last + 1 < K && subs[c.last + 1].fusedWithPrev) ++c.last;
            c.W = static_cast<long>(NB) * subs[k].laneCount;
            if (phases.empty() || subs[k].phase != subs[phases.back().chains.back().first].phase) phases.push_back(Phase());
            Phase &ph = phases.back();
            c.offset = ph.slots;
            ph.slots += (c.W + 63) / 64 * 64;
            ph.chains.push_back(c);
            k = c.last + 1;
        }
        for (auto &ph : phases)
        {
            if (ph.chains.size() == 1) ph.slots = ph.chains[0].W;
            ph.passes = (ph.slots + NT - 1) / NT;
        }

        long prefetchBudget = envInt("ACRO_HIP_PREFETCH") < 0 ? 0 : kPrefetchDoubles;
        // The first phase's own loads join the prefetch (ACRO_HIP_PREFETCH_FIRST=-1 switches that off): they are then
        // requested ahead of the later phases' inputs, and since a wavefront's loads complete in the order they were
        // issued, the first phase starts as soon as its own operands are there instead of after everything that was
        // prefetched (p=7 diffusion apply: 960 -> 943 us).  Only when some later phase prefetches at all.
        const bool firstToo = pipelined || envInt("ACRO_HIP_PREFETCH_FIRST") >= 0;
        // Later phases first (they have the latency to hide), the first phase last, with what is left of the budget.
        std::vector<size_t> phaseOrder;
        for (size_t pi = 1; pi < phases.size(); ++pi) phaseOrder.push_back(pi);
        if (firstToo && phases.size() > 1) phaseOrder.push_back(0);
        bool anyLater = false;
        for (size_t pi : phaseOrder)
        {
            // ... or on its own when its items take several passes of the workgroup: all passes request their operands
            // before the first one uses them, instead of one round trip to device memory per pass
            // (ACRO_HIP_PREFETCH_PASSES=-1 switches that off).
            // Groups of one phase keep their item loop: with everything requested up front they measured the same
            // within noise (24 streaming shapes, geometric mean 74.1 against 74.0 % of the HBM peak); the two-step
            // 27 x 27 element matrix times element vector gained, 52.8 -> 57.6 %.
            const bool severalPasses = phases[0].passes > 1 && phases.size() > 1 && envInt("ACRO_HIP_PREFETCH_PASSES") >= 0;
            if (pi == 0 && !anyLater && !pipelined && !severalPasses) break;
            Phase &ph = phases[pi];
            long perLane = 0;  // registers one lane needs: a lane serves at most one chain per pass
            bool ok = true;
            for (auto &c : ph.chains)
            {
                c.loads.assign(c.last - c.first + 1, {});
                ForwardMap forwarded;
                long perPass = 0;
                for (int kk = c.first; kk <= c.last; ++kk)
                {
                    if (subs[kk].loopMode)
                    {
                        ok = false;
                        break;
                    }
                    std::vector<std::string> scratchLines;
                    EmitUnrolledBody(kk, forwarded, scratchLines, nullptr, &c.loads[kk - c.first]);
                    perPass += static_cast<long>(c.loads[kk - c.first].size());
                }
                perLane = std::max(perLane, perPass);
            }
            if (!ok || perLane == 0 || perLane * ph.passes > prefetchBudget) continue;
            prefetchBudget -= perLane * ph.passes;
            ph.prefetched = true;
            anyLater = anyLater || pi > 0;
            // ACRO_HIP_PIPELINE=<n>: phases that hold at most n doubles per lane are carried across iterations (the
            // first phase always is: its inputs are what an iteration would otherwise start by waiting for)
            ph.carried = pipelined && (pi == 0 || perLane * ph.passes <= envInt("ACRO_HIP_PIPELINE"));
        }

        // Emits, for pass j of a phase (or for the item loop when j < 0), the selection of the chain a lane works
        // for and calls `body` inside the guarded scope of one work item.
        // A streaming group (one phase, no LDS) over few batch entries would leave most of the device idle with one
        // workgroup per entry: the passes of its item loop become workgroups of a second grid dimension instead.
        const long splitY = (phases.size() == 1 && ldsDoubles == 0 && !looped && phases[0].passes > 1 && totalGroups < 2048)
                                ? std::min<long>(phases[0].passes, 65535)
                                : 1;
        auto emitItems = [&](const Phase &ph, long j, const std::function<void(const Chain &, const std::string &)> &body) {
            std::string indent = "        ";
            if (j < 0 && splitY > 1)
                out << "    for (int w0 = tid + blockIdx.y * " << NT << "; w0 < " << ph.slots << "; w0 += " << splitY * NT
                    << ")\n    {\n";
            else if (j < 0)
                out << "    for (int w0 = tid; w0 < " << ph.slots << "; w0 += " << NT << ")\n    {\n";
            else
                out << "    {\n        const int w0 = tid + " << j * NT << ";\n";
            for (size_t ci = 0; ci < ph.chains.size(); ++ci)
            {
                const Chain &c = ph.chains[ci];
                const long end = c.offset + (ph.chains.size() == 1 ? c.W : (c.W + 63) / 64 * 64);
                if (ph.chains.size() > 1)
                {
                    out << indent << (ci ? "else if" : "if") << " (w0 < " << end << ")\n" << indent << "{\n";
                    indent += "    ";
                }
                out << indent << "const int w = w0 - " << c.offset << ";\n";
                out << indent << "if (w < " << c.W << ")\n" << indent << "{\n";
                emitHeader(subs[c.first], indent + "    ");
                std::string inner = indent + "    ";
                if (guardBatch)
                {
                    out << inner << "if (e < " << E << ")\n" << inner << "{\n";
                    inner += "    ";
                }
                body(c, inner);
                if (guardBatch) out << indent << "    }\n";
                out << indent << "}\n";
                if (ph.chains.size() > 1)
                {
                    indent.resize(indent.size() - 4);
                    out << indent << "}\n";
                }
            }
            out << "    }\n";
        };

        // Requests the prefetched inputs of one phase for the batch entries that start at the `e0` in scope.
        auto emitPrefetchLoads = [&](const Phase &ph) {
            for (long j = 0; j < ph.passes; ++j)
            {
                auto loadsOf = [&](const Chain &c, const std::string &indent) {
                    for (int kk = c.first; kk <= c.last; ++kk)
                    {
                        if (c.loads[kk - c.first].empty()) continue;
                        Body bases;
                        EmitBases(kk, bases);
                        for (const auto &l : bases.bases) out << indent << l << "\n";
                        for (const auto &ld : c.loads[kk - c.first])
                            out << indent << c.names[kk - c.first][j].at(ld.first) << " = " << ld.second << ";\n";
                    }
                };
                // A phase of one chain: lanes past the last work item request the last item's operands instead of
                // nothing.  The requests then sit in straight-line code, and the compiler can count exactly how
                // many loads were issued after the ones an earlier phase waits for (behind a branch it has to assume
                // none, and that phase would wait for everything that was prefetched).
                if (ph.chains.size() == 1 && !guardBatch && envInt("ACRO_HIP_PREFETCH_CLAMP") >= 0)
                {
                    const Chain &c = ph.chains[0];
                    out << "    {\n        const int w0 = tid + " << j * NT << ";\n";
                    out << "        const int w = w0 < " << c.W << " ? w0 : " << c.W - 1 << ";\n";
                    emitHeader(subs[c.first], "        ");
                    loadsOf(c, "        ");
                    out << "    }\n";
                    continue;
                }
                emitItems(ph, j, loadsOf);
            }
        };
        for (auto &ph : phases)
        {
            if (!ph.prefetched) continue;
            out << "    // streaming inputs of phase " << subs[ph.chains[0].first].phase
                << (pipelined ? ", held in registers across iterations\n" : ", requested before the first phase\n");
            for (auto &c : ph.chains)
                c.names.assign(c.last - c.first + 1, std::vector<std::map<std::string, std::string>>(ph.passes));
            for (long j = 0; j < ph.passes; ++j)
            {
                // One register set per pass, shared by the chains (a lane serves one chain in a pass).
                long widest = 0;
                for (auto &c : ph.chains)
                {
                    long n = 0;
                    for (int kk = c.first; kk <= c.last; ++kk)
                    {
                        for (const auto &ld : c.loads[kk - c.first])
                            c.names[kk - c.first][j][ld.first] = "pf" + str(subs[c.first].phase) + "_" + str(j) + "_" + str(n++);
                    }
                    widest = std::max(widest, n);
                }
                for (long n = 0; n < widest; ++n)
                    out << "    double pf" << subs[ph.chains[0].first].phase << "_" << j << "_" << n << " = 0.0;\n";
            }
            if (!pipelined) emitPrefetchLoads(ph);
        }
        if (pipelined)
        {
            out << "    {   // the first batch entries of this workgroup\n    const int e0 = blockIdx.x * " << NB << ";\n";
            for (const auto &ph : phases)
            {
                if (ph.carried) emitPrefetchLoads(ph);
            }
            out << "    }\n" << loopHeader;
            for (const auto &ph : phases)
            {
                if (ph.prefetched && !ph.carried) emitPrefetchLoads(ph);  // requested at the top of every iteration
            }
        }

        // results of phase `previous` that leave through their LDS tiles (after the barrier that ends it)
        auto emitCopyOut = [&](int previous) {
                for (int k = 0; k < K; ++k)
                {
                    if (subs[k].phase != previous || !CopiesOutFromLds(k)) continue;
                    const Storage &st = StoreOf(subs[k].out.uvar);
                    const bool streams = envInt("ACRO_HIP_NT_STORE") >= 0 && static_cast<long>(ldsDoubles) * 8 <= 20 * 1024;
                    out << "    {   // " << uvars[subs[k].out.uvar].name << ": LDS tiles -> device memory\n";
                    if (guardBatch)
                        out << "        const int count = (" << E << " - e0 < " << NB << " ? " << E << " - e0 : " << NB << ") * "
                            << st.tileSize << ";\n";
                    else
                        out << "        const int count = " << static_cast<long>(NB) * st.tileSize << ";\n";
                    out << "        double *dst = " << PtrName(subs[k].out.uvar) << " + e0 * " << Lit(st.tileSize) << ";\n";
                    out << "        for (int i = tid; i < count; i += " << NT << ") ";
                    if (streams)
                        out << "__builtin_nontemporal_store(lds[" << st.ldsOffset << " + i], &dst[i]);\n";
                    else
                        out << "dst[i] = lds[" << st.ldsOffset << " + i];\n";
                    out << "    }\n";
                }
        };
        bool first = true;
        for (const Phase &ph : phases)
        {
            if (!first) out << "    __syncthreads();\n";
            if (!first) emitCopyOut(subs[ph.chains[0].first].phase - 1);
            first = false;
            const long npass = ph.prefetched ? ph.passes : 1;
            for (long j = 0; j < npass; ++j)
            {
                emitItems(ph, ph.prefetched ? j : -1, [&](const Chain &c, const std::string &indent) {
                    ForwardMap forwarded;
                    for (int kk = c.first; kk <= c.last; ++kk)
                    {
                        std::vector<std::string> lines;
                        if (subs[kk].loopMode)
                            EmitLoopBody(kk, lines);
                        else
                            EmitUnrolledBody(kk, forwarded, lines, ph.prefetched ? &c.names[kk - c.first][j] : nullptr);
                        // Scopes nest (closed after the chain) so that a kernel applied in registers sees the
                        // values of its producer.
                        out << indent << "{\n";
                        for (const auto &l : lines) out << indent << "    " << l << "\n";
                    }
                    for (int kk = c.first; kk <= c.last; ++kk) out << indent << "}\n";
                });
            }
            if (ph.carried)
            {
                out << "    {   // the same inputs of this workgroup's next batch entries\n";
                out << "    const int e0_next = e0 + " << gridGroups * NB << ";\n    if (e0_next < " << E << ")\n    {\n";
                out << "    const int e0 = e0_next;\n";
                emitPrefetchLoads(ph);
                out << "    }\n    }\n";
            }
        }
        {
            bool lastCopies = false;
            for (int k = 0; k < K; ++k) lastCopies = lastCopies || (subs[k].phase == subs.back().phase && CopiesOutFromLds(k));
            if (lastCopies)
            {
                out << "    __syncthreads();\n";
                emitCopyOut(subs.back().phase);
            }
        }
        if (looped && ldsDoubles > 0) out << "    __syncthreads();\n";
        out << "    }\n}\n";

        plan.source = out.str();
        HipLaunch launch;
        launch.function_name = function_name;
        launch.grid = static_cast<unsigned>(gridGroups);
        launch.grid_y = static_cast<unsigned>(splitY);
        launch.block = static_cast<unsigned>(NT);
        for (int si = 0; si < NumParamStores(); ++si) launch.params.push_back(si);
        for (int g = 0; g < NumGatherSlots(); ++g)
        {
            launch.params.push_back(-2 - 2 * g);
            launch.params.push_back(-3 - 2 * g);
        }
        plan.gathers_applied = NumGatherSlots() > 0;
        plan.launches.push_back(launch);
        plan.nb = NB;
        plan.lds_bytes = ldsDoubles * 8;
        FillParams(plan, true);
        for (const auto &s : subs)
        {
            if (s.out.repeated && s.op == '=')
                plan.zero_fills.push_back({uvars[s.out.uvar].storage, uvars[s.out.uvar].viewOffset, s.out.size});
        }
    }
};

}  // namespace

HipKernelPlan GenerateHipKernel(const DimensionedMultiKernel &mk, const HipCodegenOptions &options)
{
    // Partial results of a reordered kernel may take up to 48 KB of LDS per batch entry; when the tiles that are
    // live together do not fit in a workgroup's 64 KB, plan again with tiles of half that size (any two fit), and
    // finally evaluate the kernel as written.
    for (long maxTile : {6144L, 3072L})
    {
        Generator g(mk, options, maxTile);
        HipKernelPlan plan = g.Run();
        if (!g.factorisationAbandoned) return plan;
    }
    Generator g(mk, options, 0);
    return g.Run();
}

}  // namespace acro
