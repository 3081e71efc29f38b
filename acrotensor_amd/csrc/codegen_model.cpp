// Kernel code generator, the model of a kernel group: operands, storages and views, what each kernel reads of what earlier kernels wrote, contraction ordering.
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

auto Generator::BuildModel() -> void
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

auto Generator::NonBatchVolume(const std::set<int> &ids) const -> double
{
    double v = 1.0;
    for (int id : ids)
    {
        if (id != batch) v *= extent[id];
    }
    return v;
}

auto Generator::FactoriseSearch(const Sub &orig, std::vector<int> &live, std::vector<std::vector<int>> &idxOf, std::vector<int> &remaining, double cost, std::vector<FactorStep> &steps, double &best, long &bestSlowest, std::vector<FactorStep> &bestSteps, long &visits) const -> void
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
auto Generator::FactoriseKernels() -> void
{
    std::vector<Sub> expanded;
    int counter = 0;
    for (size_t ki = 0; ki < subs.size(); ++ki)
    {
        if (subs.size() == 1 && ProductThenRowSums(static_cast<int>(ki), subs[ki], expanded, counter)) continue;
        if (FactoriseKernel(static_cast<int>(ki), subs[ki], subs.size() == 1, expanded, counter)) continue;
        if (subs.size() == 1 && StageReusedOperands(static_cast<int>(ki), subs[ki], expanded, counter)) continue;
        expanded.push_back(subs[ki]);
    }
    subs.swap(expanded);
}

// A kernel on its own whose per-entry operands are small and read many times over by the lanes of the entry (batched
// matrix products "A_e_i_j = B_e_i_k C_e_k_j" with 16 x 16 matrices: every value 16 times, 32 loads per output
// straight from device memory, lanes a row or a column apart: 28 % of the HBM peak) copies those operands to LDS tiles
// first, with the lanes along the operand as it lies in memory, and computes from the tiles.  The copies are steps of
// the generator's own ("_S1_e_i_k = B_e_i_k"), placed, fused and emitted like the steps of a reordered kernel.
auto Generator::StageReusedOperands(int ki, const Sub &asWritten, std::vector<Sub> &result, int &counter) -> bool
{
    if (envInt("ACRO_HIP_STAGE_ENTRIES") < 0 || batch < 0 || !opt.noalias || asWritten.contr.empty() || asWritten.matrixOp != 0) return false;
    Sub orig = asWritten;
    if (orig.out.repeated || orig.in.size() < 2 || NumGatherSlots() > 0) return false;
    {
        ProductShape onMatrixCores;  // products of larger element matrices have a schedule of their own
        if (ProductPattern(asWritten, onMatrixCores)) return false;
    }
    const long outputs = product(orig.outIdx, extent) / extent[batch];
    const long stageMost = envInt("ACRO_HIP_STAGE_MOST", 8000);
    if (outputs < 4 || outputs > stageMost / 2) return false;
    // Tiny matrices (fewer than 64 outputs) are staged as well (3 x 3: 64 -> 82 %, 5 x 5: 46 -> 77 %, 6 x 6: 48 -> 80 %,
    // 7 x 7: 46 -> 77 % of the HBM peak, with some 500 outputs per workgroup of 256 lanes), except those with fewer than
    // 16 outputs whose operands' entries are all powers of two of doubles: those lie in whole lines and the lanes read
    // them as well from device memory (with the launches rotated over tensors that no cache holds: 2 x 2 times 2 x 8
    // 77 % straight and 68 % staged, 2 x 8 times 8 x 4 70 and 69 %, 2 x 2 times 2 x 2 75 and 76 %; from 16 outputs on
    // the tiles win: 4 x 4 times 4 x 4 61 -> 76 %, 4 x 2 times 2 x 4 68 -> 76 %, 8 x 2 times 2 x 2 73 -> 77 %).
    const bool tiny = outputs < 64;
    const long wholeLinesFrom = envInt("ACRO_HIP_STAGE_WHOLE_LINES", 16);  // -1: never
    bool wholeLines = true;
    std::vector<char> staged(orig.in.size(), 0);
    long total = 0;
    int count = 0;
    for (size_t v = 0; v < orig.in.size(); ++v)
    {
        const VarRef &r = orig.in[v];
        if (r.repeated || r.uvar == orig.out.uvar || r.idx.empty() || r.idx[0] != batch) continue;
        bool again = false;  // the same tensor twice: one tile would do, keep it simple
        for (size_t w = 0; w < orig.in.size(); ++w) again = again || (w != v && orig.in[w].uvar == r.uvar);
        if (again) continue;
        const long perEntry = r.size / extent[batch];
        // how many outputs each value goes into: the output indices that the operand does not carry
        long reads = 1;
        for (int id : orig.outIdx) reads *= (id == batch || has(r.idx, id)) ? 1 : extent[id];
        wholeLines = wholeLines && (perEntry & (perEntry - 1)) == 0;
        if (perEntry < (tiny ? 4 : 16) || perEntry > stageMost / 2 || reads < (tiny ? 2 : 8)) continue;
        staged[v] = 1;
        total += perEntry;
        ++count;
    }
    // Two such operands: products of element matrices.  With one (an element vector under an element matrix, the
    // vectors of a dense operator) the kernel has schedules of its own that read the big operand once and well.
    if (count < 2 || total > stageMost || (tiny && wholeLines && (wholeLinesFrom < 0 || outputs < wholeLinesFrom))) return false;
    // More than 1 024 outputs or 2 048 staged values per entry (products of 33 x 33 to 62 x 62 matrices, which the lanes
    // read straight from device memory at 9 - 12 % of the HBM peak: staged 49 - 66 %): only the two factors of a
    // product, each of which carries a contracted index
    if (outputs > 1024 || total > 2048)
    {
        bool factors = count == 2;
        for (size_t v = 0; v < orig.in.size(); ++v)
        {
            bool contracted = false;
            for (int id : orig.in[v].idx) contracted = contracted || has(orig.contr, id);
            factors = factors && (!staged[v] || contracted);
        }
        if (!factors) return false;
    }
    // (tiny entries under one shared operator, "A_e_i = B_i_j X_e_j W_e D_e_j", belong to the operator schedule)
    int operators = 0;
    for (const auto &r : orig.in)
    {
        bool contracted = false, free = false;
        for (int id : r.idx) (has(orig.contr, id) ? contracted : free) = true;
        operators += (!has(r.idx, batch) && contracted && free) ? 1 : 0;
    }
    if (tiny && operators == 1) return false;
    // (the same for vectors of any length with pointwise factors of their shape, "A_e_i = B_i_j X_e_j D_e_j")
    bool vectorsOnly = true;
    for (size_t v = 0; v < orig.in.size(); ++v)
    {
        if (!staged[v]) continue;
        for (int id : orig.in[v].idx) vectorsOnly = vectorsOnly && (id == batch || !has(orig.outIdx, id));
    }
    if (operators == 1 && vectorsOnly) return false;
    // With one output per lane every multiply-add reads both of its factors from LDS, and LDS bounds the kernel
    // (24 x 24 products: 48 % of the HBM peak, 30 x 30: 35 %).  A lane that owns a 2 x 2 block of outputs reads half
    // as much.  Register tiles are whole indices, so an output index of even extent is split in two, "i = 2 i' + i''"
    // (extent divisible by three only: in three), in every operand, which describes the same memory with one
    // dimension more, and the halves i'' become the tile (24 x 24: 83 %, 30 x 30: 80 %, 12 x 12: 72 -> 89 %).
    std::vector<int> blockIdx;
    bool splittable = !tiny && envInt("ACRO_HIP_STAGE_ENTRIES") < 2;
    for (size_t v = 0; v < orig.in.size(); ++v)
    {
        const int u = orig.in[v].uvar;
        for (size_t w = 0; w < orig.in.size(); ++w) splittable = splittable && (w == v || orig.in[w].uvar != u);
        splittable = splittable && u != orig.out.uvar;
    }
    // (every operand must be a whole tensor of its own: its storage is then described by the split dimensions)
    auto wholeTensor = [&](const VarRef &r) {
        if (static_cast<size_t>(r.uvar) >= opt.views.size()) return true;
        const HipOperandView &view = opt.views[r.uvar];
        long entries = 1;
        for (int d : view.root_dims) entries *= d;
        bool shared = false;
        for (size_t u = 0; u < opt.views.size(); ++u)
            shared = shared || (static_cast<int>(u) != r.uvar && opt.views[u].storage >= 0 && opt.views[u].storage == view.storage);
        return view.storage < 0 || (!shared && view.offset == 0 && (view.root_dims.empty() || entries == r.size));
    };
    splittable = splittable && wholeTensor(orig.out);
    for (const auto &r : orig.in) splittable = splittable && wholeTensor(r);
    if (splittable)
    {
        const std::vector<int> outputIds = orig.outIdx;
        for (int id : outputIds)
        {
            if (id == batch || extent[id] < 4) continue;
            int t = extent[id] % 2 == 0 ? 2 : (extent[id] % 3 == 0 ? 3 : (extent[id] % 5 == 0 && envInt("ACRO_HIP_SPLIT_FIVE") >= 0 ? 5 : 1));
            if (t == 5)
            {
                // blocks of five only while a hundred lane items are left per entry (25 x 25 in 5 x 5 blocks: 25 items,
                // two waves in eight busy, 49 % of the HBM peak)
                long items = 1;
                for (int other : orig.outIdx) items *= (other == batch || has(blockIdx, other)) ? 1 : extent[other];
                if (items / 5 < envInt("ACRO_HIP_SPLIT_FIVE_ITEMS", 100)) t = 1;
            }
            if (t == 1) continue;
            // two new loop indices, named after the old one
            auto fresh = [&](std::string name) {
                while (std::find(idxName.begin(), idxName.end(), name) != idxName.end()) name += "x";
                return name;
            };
            const int hi = nidx, lo = nidx + 1;
            nidx += 2;
            idxName.push_back(fresh(idxName[id] + "hi"));
            extent.push_back(extent[id] / t);
            idxName.push_back(fresh(idxName[id] + "lo"));
            extent.push_back(t);
            auto splitRef = [&](VarRef &r) {
                VarRef n = r;
                n.idx.clear();
                n.ext.clear();
                n.stride.clear();
                for (size_t d = 0; d < r.idx.size(); ++d)
                {
                    if (r.idx[d] != id)
                    {
                        n.idx.push_back(r.idx[d]);
                        n.ext.push_back(r.ext[d]);
                        n.stride.push_back(r.stride[d]);
                        continue;
                    }
                    n.idx.push_back(hi);
                    n.ext.push_back(r.ext[d] / t);
                    n.stride.push_back(r.stride[d] * t);
                    n.idx.push_back(lo);
                    n.ext.push_back(t);
                    n.stride.push_back(r.stride[d]);
                }
                r = n;
            };
            splitRef(orig.out);
            for (auto &r : orig.in) splitRef(r);
            std::vector<int> ids;
            for (int o : orig.outIdx)
            {
                if (o != id) ids.push_back(o);
                else
                {
                    ids.push_back(hi);
                    ids.push_back(lo);
                }
            }
            orig.outIdx = ids;
            blockIdx.push_back(lo);
        }
        if (!blockIdx.empty())
        {
            reshaped.insert(orig.out.uvar);
            for (const auto &r : orig.in) reshaped.insert(r.uvar);
        }
    }
    DimensionedKernel *kernel = mk.Kernels[ki];
    auto refText = [&](const std::string &name, const std::vector<int> &ids) {
        std::string t = name;
        for (int id : ids) t += "_" + idxName[id];
        return t;
    };
    Sub fin = orig;
    std::string finText = refText(kernel->GetVarName(-1), orig.out.idx) + " " + (orig.op == '=' ? "=" : std::string(1, orig.op) + "=");
    for (size_t v = 0; v < orig.in.size(); ++v)
    {
        const VarRef &r = orig.in[v];
        if (!staged[v])
        {
            finText += " " + refText(kernel->GetVarName(static_cast<int>(v)), r.idx);
            continue;
        }
        UVarInfo info;
        info.isVirtual = true;
        info.isStagedCopy = true;
        info.name = "_S" + str(static_cast<long>(++counter));
        VarRef res;
        res.uvar = static_cast<int>(uvars.size());
        res.idx = r.idx;
        res.ext = r.ext;
        res.stride = r.stride;
        res.size = r.size;
        // The factor that carries the last output index with a contracted index as its fastest dimension ("A_e_i_j =
        // B_e_i_k C_e_j_k": C): neighbouring lanes would read its copy a row apart.  The copy is laid out with the
        // contracted indices in front instead, so that they read neighbouring values as they do for "C_e_k_j"
        // (12 x 12: 82 -> 87 % of the HBM peak, 24 x 24 72 -> 82 %, 40 x 40 46 -> 58 %); the lanes of the copying step still follow the operand in memory.
        if (envInt("ACRO_HIP_STAGE_TRANSPOSED") >= 0 && !orig.outIdx.empty() && has(r.idx, orig.outIdx.back()) && has(orig.contr, r.idx.back()) &&
            r.idx[0] == batch)
        {
            std::vector<size_t> order(1, 0);
            for (size_t d = 1; d < r.idx.size(); ++d)
            {
                if (has(orig.contr, r.idx[d])) order.push_back(d);
            }
            for (size_t d = 1; d < r.idx.size(); ++d)
            {
                if (!has(orig.contr, r.idx[d])) order.push_back(d);
            }
            res.idx.clear();
            res.ext.clear();
            for (size_t d : order)
            {
                res.idx.push_back(r.idx[d]);
                res.ext.push_back(r.ext[d]);
            }
            res.stride.assign(order.size(), 1);
            for (size_t d = order.size() - 1; d-- > 0;) res.stride[d] = res.stride[d + 1] * res.ext[d + 1];
        }
        uvars.push_back(info);
        Sub copy;
        copy.op = '=';
        copy.out = res;
        copy.outIdx = r.idx;
        copy.in.assign(1, r);
        copy.contrCount = 1;
        copy.flatItems = true;
        copy.text = refText(info.name, res.idx) + " = " + refText(kernel->GetVarName(static_cast<int>(v)), r.idx);
        result.push_back(copy);
        fin.in[v] = res;
        finText += " " + refText(info.name, res.idx);
    }
    fin.text = finText + "   (operands staged in LDS: " + orig.text + ")";
    fin.wantedTile = blockIdx;
    result.push_back(fin);
    factorised = true;
    return true;
}

// An element matrix applied to an element vector, "A_e_i = B_e_i_j C_e_j", whose rows are not a multiple of four
// doubles long (27 x 27): with the lanes along the rows, whether one lane or a few per row, a wavefront reads its
// matrices in pieces of a row, 216 bytes apart (47 - 53 % of the HBM peak).  Evaluated in two steps instead: the
// products "_F1_e_i_j = B_e_i_j C_e_j" with the lanes along the matrix as it lies in memory, into a tile in LDS,
// then the sums over j, one lane per row (a row stride that is odd spreads the lanes over the banks).
auto Generator::ProductThenRowSums(int ki, const Sub &orig, std::vector<Sub> &result, int &counter) -> bool
{
    if (envInt("ACRO_HIP_ROW_SUMS") < 0 || batch < 0 || orig.in.empty() || orig.in.size() > 3 || orig.contr.empty() || !opt.noalias) return false;
    if (orig.out.repeated || orig.matrixOp != 0) return false;
    {
        ProductShape onMatrixCores;  // (the product schedule takes matrices of up to 128 x 128 with such rows)
        if (ProductPattern(orig, onMatrixCores)) return false;
    }
    const VarRef *matrix = nullptr;
    std::vector<const VarRef *> vecs;
    for (const auto &r : orig.in)
    {
        if (r.repeated || r.uvar == orig.out.uvar) return false;
        bool all = has(r.idx, batch);
        for (int id : orig.outIdx) all = all && has(r.idx, id);
        for (int id : orig.contr) all = all && has(r.idx, id);
        if (all && matrix == nullptr)
            matrix = &r;
        else
            vecs.push_back(&r);
    }
    if (matrix == nullptr) return false;
    // the contraction indices are the matrix's fastest dimensions, the vectors carry nothing but them and the batch
    const size_t nc = orig.contr.size();
    if (matrix->idx.size() < nc + 1 || matrix->idx[0] != batch) return false;
    bool contractedLast = true;
    for (size_t d = 0; d < nc; ++d) contractedLast = contractedLast && has(orig.contr, matrix->idx[matrix->idx.size() - 1 - d]);
    // (the other way round, a vector applied from the left to an element matrix of few columns, "A_e_j = B_e_i_j C_e_i":
    // the lanes of the second step add down the columns of the tile)
    const bool columns = !contractedLast;
    if (!contractedLast && !columns) return false;
    for (const VarRef *vec : vecs)
    {
        for (int id : vec->idx)
        {
            if (id != batch && !has(orig.contr, id)) return false;
        }
        // (factors along part of a row, "A_e = B_e_i_j C_i D_j": no gain from HBM, 67 -> 50 % re-launched)
        for (int id : orig.contr)
        {
            if (vecs.size() > 1 && !has(vec->idx, id)) return false;
        }
    }
    const long rows = product(orig.outIdx, extent) / extent[batch], row = orig.contrCount;
    if (rows * row > 4096 || row > 512) return false;
    if (columns)
    {
        // (up to four columns of 16 - 128 rows, every factor with the batch index; from HBM 27 x 2 46 -> 73 %, 64 x 2
        // 52 -> 73 %, 64 x 3 54 -> 69 %, 27 x 4 57 -> 67 %, 16 x 2 65 -> 76 %, sums of 64 x 2 without a vector 63 -> 69 %; with a
        // vector that all entries share 63 -> 46 %)
        if (rows > 4 || row < 16 || row > 128) return false;
        for (const VarRef *vec : vecs)
        {
            if (!has(vec->idx, batch)) return false;
        }
        for (int id : orig.contr)
        {
            for (size_t d = 0; d < matrix->idx.size(); ++d)
            {
                if (matrix->idx[d] == id && d + 1 == matrix->idx.size()) return false;   // (mixed: neither rows nor columns)
            }
        }
    }
    else if (rows >= 4)
    {
        if (row % 4 == 0 || row < 9 || vecs.size() != 1) return false;
    }
    else
    {
        // One to three sums per entry ("A_e = B_e_i C_e_i", "A_e = B_e_i", "A_e_k = B_e_k_i C_e_i" with two components), from
        // HBM: rows of 9 doubles 51 -> 79 % of the HBM peak, 15: 63 -> 77 %, 20: 65 -> 77 %, 27: 57 -> 77 %, 45: 64 -> 75 %,
        // dot products of rows of 9: 59 -> 77 %, of 27: 62 -> 76 %; rows of 3 and 5 lose (75 -> 56 %, 73 -> 67 %), 6 and
        // powers of two neither gain nor lose, rows of 100 lose (79 -> 76 %).
        if (row < 7 || row > 64 || (row & (row - 1)) == 0) return false;
        // (a factor that all entries share is read by every lane of the first step through its own index: with short rows
        // that costs more than the lanes along the rows lose, from HBM "A_e = B_e_i C_i" with rows of 7 74 -> 58 %, "A_e =
        // B_i C_i D_e_i" with rows of 12 64 -> 52 %; rows of 20 and 27 gain, 56 -> 59 % and 47 -> 60 %)
        for (const VarRef *vec : vecs)
        {
            if (!has(vec->idx, batch) && row < 20) return false;
        }
    }

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
auto Generator::FactoriseKernel(int ki, const Sub &orig, bool alone, std::vector<Sub> &result, int &counter) -> bool
{
    const int nin = static_cast<int>(orig.in.size());
    // (two operands: only where an operand carries a contraction index alone, "A_e = B_e_j C_e_i", and can be summed over
    // it before the product; the search finds nothing to do otherwise)
    if (batch < 0 || nin < (envInt("ACRO_HIP_FACTORISE_PAIRS") < 0 ? 3 : 2) || orig.contr.empty() || !opt.noalias || orig.out.repeated) return false;
    if (alone && ReductionServes(orig)) return false;  // the reduction schedule serves it
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
    // (a product of two operands that can be summed first repeats its loads for every term as written, every lane along
    // rows of its own: "A_e = B_e_j C_e_i" with 32 and 27 terms took 6.0 ms for 500 MB; such a kernel is taken apart from
    // 256 multiply-adds per entry on where that leaves an eighth of them)
    const bool worthIt = nin == 2 ? asWritten >= 256.0 && best * 8.0 <= asWritten
                                  : asWritten >= kFactoriseMinWork && best * kFactoriseMinGain <= asWritten;
    if (!eager && !worthIt) return false;

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

auto Generator::BuildStorages() -> void
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
        const bool hasView = static_cast<size_t>(u) < opt.views.size() && !opt.views[u].root_dims.empty() && reshaped.count(u) == 0;
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
auto Generator::Covered(const Storage &st, const std::vector<int> &fixed, const std::vector<std::vector<int>> &written) const -> bool
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

auto Generator::AnalyseCoverage() -> void
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

auto Generator::CheckFusable(std::string &why) -> bool
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

}  // namespace codegen
}  // namespace acro
