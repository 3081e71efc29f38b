// Kernel code generator, code of one work item: offsets, operand sources, unrolled / looped / lane-shared / matrix bodies, stores.
#include "hip_codegen_impl.hpp"

namespace acro
{
namespace codegen
{

// Pair number of an operand that is read through an index map instead of from its own memory, or -1.
auto Generator::GatherSlot(int uvar) const -> int
{
    return static_cast<size_t>(uvar) < opt.gathered.size() ? opt.gathered[uvar] : -1;
}

auto Generator::NumGatherSlots() const -> int
{
    int n = 0;
    for (int g : opt.gathered) n = std::max(n, g + 1);
    return n;
}

// Read of entry `offset` of an operand from device memory.
auto Generator::GlobalRead(int uvar, const std::string &offset, bool streamedOnce) const -> std::string
{
    const int g = GatherSlot(uvar);
    if (g < 0 && streamedOnce) return "__builtin_nontemporal_load(&" + PtrName(uvar) + "[" + offset + "])";
    if (g < 0) return PtrName(uvar) + "[" + offset + "]";
    // (the map read with the non-temporal hint: scatter + p=3 mass apply in one launch 90.4 -> 92.9 us from HBM, not taken)
    return "G" + str(g) + "s[G" + str(g) + "m[" + offset + "]]";
}

// LDS stride of a view dimension, and the constant LDS offset of the view inside the storage's tile
auto Generator::LdsStride(int uvar, size_t d) const -> int
{
    const UVarInfo &op = uvars[uvar];
    return StoreOf(uvar).ldsStride[d + op.fixed.size()];
}

auto Generator::LdsViewOffset(int uvar) const -> long
{
    const UVarInfo &op = uvars[uvar];
    long off = 0;
    for (size_t d = 0; d < op.fixed.size(); ++d) off += static_cast<long>(op.fixed[d]) * StoreOf(uvar).ldsStride[d];
    return off;
}

// Offset of an occurrence split into a run-time part (batch entry + lane indices) and, for a given
// assignment of tile / contraction indices, a literal part.
auto Generator::RuntimeOffset(const VarRef &r, const Sub &s, bool lds) const -> std::string
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

auto Generator::LiteralOffset(const VarRef &r, const Sub &s, bool lds, const std::vector<int> &value) const -> long
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

auto Generator::SourceOf(int k, int v) const -> Source
{
    const Sub &s = subs[k];
    const VarRef &r = s.in[v];
    if (FromRegisters(k, v)) return kFromRegisters;
    if (StoreOf(r.uvar).inLds && (readCovered[k][v] || StoreOf(r.uvar).staged)) return kFromLds;
    if (IsUniform(s, r, s.tile)) return kFromConstant;
    return kFromGlobal;
}

// Batch part of a scalar operand's address ("e0 * stride + ", e0 being uniform) or nothing.
auto Generator::ScalarBase(const VarRef &r) const -> std::string
{
    std::string base;
    for (size_t d = 0; d < r.idx.size(); ++d)
    {
        if (r.idx[d] == batch) base += "e0 * " + Lit(r.stride[d]) + " + ";
    }
    return base;
}

// Device-memory operand whose values are read once each, by lanes that follow it through memory so that every load
// instruction of a wavefront takes whole 128-byte lines: requested with the non-temporal hint, which keeps lines that
// nothing reads again from displacing others (from HBM: "A_e_i = B_e_i C_e_i D_e_i" 345 -> 319 us, "A_e = B_e_n" with
// rows of 1 024 92 -> 84 us, "A_e_i = B_e_i_n" 182 -> 161 us).  Not where lanes read pieces of lines that a later
// instruction or a neighbouring workgroup completes: those lines are then fetched twice (the p=3 mass apply 87 -> 106 us,
// the p=7 diffusion apply 939 -> 1 626 us with every streaming operand read that way).
auto Generator::StreamedOnce(int k, int v) const -> bool
{
    if (envInt("ACRO_HIP_NT_LOADS") < 0 || batch < 0) return false;
    const Sub &s = subs[k];
    const VarRef &r = s.in[v];
    if (SourceOf(k, v) != kFromGlobal || !IsPureInput(r.uvar) || GatherSlot(r.uvar) >= 0 || r.repeated || r.idx.empty() || r.idx[0] != batch) return false;
    if (s.matrixOp != 0 || entriesFastest) return false;
    if (((r.size / E) * NB) % 16 != 0) return false;   // the share of a workgroup: whole lines
    // (a launch that writes more than it reads has few loads to hide behind its stores, and the hinted load takes longer to
    // come back: "A_e_j_i = B_e_i C_j_i" with 6 values read and 42 written per entry 42 -> 73 us, "A_e_i_j_k = B_i_j_k
    // C_e_i_k" 89 -> 135 us from HBM)
    if (WritesDominate()) return false;
    // (a contraction that runs as a counted loop loads its operands anew in every turn: an operand that does not carry
    // every contraction index would be asked for again and again, "A_e_j += B_l_k_i C_e_i_j": 1.8 -> 3.3 ms)
    if (s.loopMode)
    {
        for (int id : s.contr)
        {
            if (!has(r.idx, id)) return false;
        }
    }
    // (read by this kernel only: a second kernel of the group would ask for lines that the hint has let go)
    int readers = 0;
    for (const auto &other : subs)
    {
        for (const auto &o : other.in) readers += o.uvar == r.uvar ? 1 : 0;
    }
    if (readers != 1) return false;
    if (s.splitLanes > 0)
    {
        if (!s.tile.empty()) return false;
        // the lanes of an output walk along the contraction, which is the operand's fastest dimensions in the kernel's order
        // and long enough for a row of 16 lanes to take a line per step; every output has a row of its own
        const size_t nc = s.contr.size();
        if (s.contrCount % 16 != 0 || r.idx.size() < nc + 1 || !std::equal(s.contr.begin(), s.contr.end(), r.idx.end() - static_cast<long>(nc))) return false;
        for (int id : s.outIdx)
        {
            if (!has(r.idx, id)) return false;
        }
        return true;
    }
    // The lanes of an entry number the operand's fastest dimensions in its own order, so that they read consecutive
    // values and no value goes to two work items (tile and contraction indices are loops of the work item: one load
    // instruction each).  Either the operand has no other dimensions, the lanes of neighbouring entries then continue the
    // run ("A_e_i = B_e_i C_e_i D_e_i", the products of "A_e = B_e_i C_e_i" with rows of 27), or the run of an entry is whole
    // lines and so is the entry ("T_e_q_j_k = B_q_i X_e_i_j_k" with 4 x 4 x 4 values per entry and the lanes on (j, k): with
    // the element vector of the p=3 mass apply read that way the launch re-run on its tensors takes 79.1 instead of 86.9 us,
    // the geometric factors staying in the memory-side cache, and 85.4 instead of 87.4 us from HBM).
    const size_t nl = s.lane.size();
    if (nl == 0 || r.idx.size() < nl + 1 || !std::equal(s.lane.begin(), s.lane.end(), r.idx.end() - static_cast<long>(nl))) return false;
    if (r.idx.size() == nl + 1) return true;
    return s.laneCount % 16 == 0 && (r.size / E) % 16 == 0;
}

// Device-memory operand that a phase may load long before it is used: never written by the group and
// addressed through the batch index (the streaming inputs, not small tables).
auto Generator::Prefetchable(int k, int v) const -> bool
{
    const VarRef &r = subs[k].in[v];
    return SourceOf(k, v) == kFromGlobal && IsPureInput(r.uvar) && has(r.idx, batch);
}

auto Generator::OperandExpr(int k, int v, const std::vector<int> &value, Body &body, const ForwardMap &forwarded) -> std::string
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
        const std::string rhs = GlobalRead(r.uvar, base + " + " + Lit(off), StreamedOnce(k, v));
        body.loads.push_back("const double " + name + " = " + rhs + ";");
        if (Prefetchable(k, v)) body.globalLoads.push_back(std::make_pair(key, rhs));
    }
    body.loadMemo[key] = name;
    return name;
}

// Sum over the contraction indices deeper than `depth`, of the product of the factors that close at those
// levels.  Returns the name of a temporary, or "" when the remaining sum is exactly one.
auto Generator::PartialSum(int k, int depth, std::vector<int> &value, Body &body, const std::vector<int> &level, const ForwardMap &forwarded) -> std::string
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

auto Generator::EmitBases(int k, Body &body) -> void
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

// The store of kernel k's output to device memory is dead when a later kernel of the group rewrites the same
// view completely, takes the old value from the LDS tile (or does not need it), and every read in between is
// served from the tile as well.
auto Generator::StoreIsDead(int k) const -> bool
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

// A result that no later kernel of the launch reads back from device memory is written with a non-temporal
// store: it streams to HBM without displacing the operands that the strided loads of other lanes still need in
// the caches (measured +2.5 % on the p=3 mass apply; non-temporal LOADS measured -20 % and are not used).
// Such stores complete later, which delays the retirement of the workgroup: where LDS allows only a few resident
// workgroups per CU that costs more than it gains (p=7 diffusion apply, 3 workgroups per CU: -14 %), so they are
// only used while at least 8 workgroups fit.
// They also get less write combining, so they are only used when one store instruction of a wavefront fills at
// least about half of every 128-byte line it touches (scattered 8-byte pieces written this way measured 1.7x
// slower than ordinary stores).
auto Generator::StreamsOut(int k) const -> bool
{
    if (envInt("ACRO_HIP_NT_STORE") < 0) return false;
    if (static_cast<long>(ldsDoubles) * 8 > 20 * 1024 && envInt("ACRO_HIP_NT_STORE") < 2) return false;
    const double coverage = WaveStoreLineCoverage(k);
    if (coverage < 0.45) return false;
    // Lines filled in part and a launch that writes more to device memory than it reads: ordinary stores (single-kernel
    // 3D interpolation "U_e_q_r_s = B_q_i B_r_j B_s_k X_e_i_j_k", runs of 200 bytes: 59 % of the HBM peak non-temporal,
    // 78 % ordinary).  Read-dominated launches keep them (products of 8 x 8 to 24 x 24 element matrices in 2 x 2 blocks,
    // 73 % of the lines filled: 84 % against 72 %), and so do whole lines (outer product 87 against 46 %).
    if (coverage < 0.95 && WritesDominate()) return false;
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

// Does the launch write more to device memory than it reads from it (per batch entry)?
auto Generator::WritesDominate() const -> bool
{
    if (batch < 0) return false;
    double stored = 0.0, loaded = 0.0;
    std::set<int> counted;
    for (int k = 0; k < static_cast<int>(subs.size()); ++k)
    {
        const Sub &s = subs[k];
        if (StoresToGlobal(k)) stored += static_cast<double>(s.out.size) / static_cast<double>(E);
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            const Source src = SourceOf(k, static_cast<int>(v));
            if ((src == kFromGlobal || src == kFromConstant) && has(s.in[v].idx, batch) && counted.insert(s.in[v].uvar).second)
                loaded += static_cast<double>(s.in[v].size) / static_cast<double>(E);
        }
    }
    return stored > loaded;
}

// How much of the 128-byte lines that one store instruction of kernel k touches does it fill, on average over
// the instructions of the first wavefront?  A lane's stores to consecutive addresses are counted as one
// instruction per pair of doubles (the compiler merges them into 16-byte stores).
auto Generator::WaveStoreLineCoverage(int k, int entries) const -> double
{
    const Sub &s = subs[k];
    // (entries > 0: for that many batch entries per workgroup instead of the number chosen, for use before it is)
    const long items = std::min<long>(64, static_cast<long>(entries > 0 ? entries : NB) * s.laneCount);
    std::vector<std::vector<long>> perLane(items);
    for (long w = 0; w < items; ++w)
    {
        std::vector<int> value(nidx, 0);
        // (numbered with the entry fastest: neighbouring lanes take neighbouring entries of one lane item)
        const long perGroup = entries > 0 ? entries : NB;
        long rest = entriesFastest ? (w / perGroup) % s.laneCount : w % s.laneCount;
        for (int j = static_cast<int>(s.lane.size()) - 1; j >= 0; --j)
        {
            value[s.lane[j]] = static_cast<int>(rest % extent[s.lane[j]]);
            rest /= extent[s.lane[j]];
        }
        if (batch >= 0) value[batch] = static_cast<int>(entriesFastest ? w % perGroup : w / s.laneCount);
        const long tiles = s.tileCount;
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

auto Generator::GlobalStore(int k, const std::string &gaddr, const std::string &value) const -> std::string
{
    if (StreamsOut(k)) return "__builtin_nontemporal_store(" + value + ", &" + gaddr + ");";
    return gaddr + " = " + value + ";";
}

auto Generator::NeedsLdsCopy(int k) const -> bool
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
auto Generator::CopiesOutFromLds(int k) const -> bool
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
auto Generator::EmitUnrolledBody(int k, ForwardMap &forwarded, std::vector<std::string> &lines, const std::map<std::string, std::string> *preloaded, std::vector<std::pair<std::string, std::string>> *globalLoads) -> void
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
auto Generator::EmitMatrixBody(int k, Body &body, ForwardMap &forwarded) -> void
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
// Lanes that share a contraction take its terms two at a time when the one contraction index is the fastest
// dimension of every operand that carries it: one 16-byte load per operand and pair instead of two 8-byte loads (a
// matrix of 2^20 rows of 64 times a shared vector: 59.8 % of the HBM peak with single terms; see the schedule comment
// of the generated kernel for what it takes now).  ACRO_HIP_SPLIT_PAIRS=-1 switches that off.
auto Generator::SplitLanesTakePairs(int k) const -> bool
{
    const Sub &s = subs[k];
    if (s.splitLanes <= 0 || envInt("ACRO_HIP_SPLIT_PAIRS") < 0 || s.contr.empty()) return false;
    // (several contraction indices: the pairs run along the last one, which the flattened range walks fastest; its
    // extent is even, so the two terms of a pair share all the other indices.  "A_e = B_e_i_j C_i D_j": 56 -> 66 %.)
    const int fastest = s.contr.back();
    if (extent[fastest] % 2 != 0 || s.contrCount < 2L * s.splitLanes) return false;
    // Long rows stream better term by term, eight 8-byte loads in flight per lane (rows of 1 024: 75.3 against 73.5 % of
    // the HBM peak, four rows of 256: 76.6 against 74.7 %); the pairs pay where a lane has few terms (16 x 16 element
    // matrix times vector 69.3 -> 76.4 %, 64 x 64 71.0 -> 72.0 %).
    if (s.contrCount > 8L * s.splitLanes) return false;
    bool any = false;
    for (size_t v = 0; v < s.in.size(); ++v)
    {
        const VarRef &r = s.in[v];
        if (!has(r.idx, fastest)) continue;
        const Source src = SourceOf(k, static_cast<int>(v));
        if ((src != kFromGlobal && src != kFromConstant) || GatherSlot(r.uvar) >= 0 || r.repeated) return false;
        if (r.idx.back() != fastest || r.stride.back() != 1) return false;
        any = true;
    }
    return any;
}

// One output per batch entry, its contraction shared by s.splitLanes adjacent lanes.
auto Generator::EmitSplitLanesBody(int k, std::vector<std::string> &lines) -> void
{
    const Sub &s = subs[k];
    Body body;
    EmitBases(k, body);
    const int L = s.splitLanes;
    lines.push_back("// " + s.text + "   (contraction shared by " + str(L) + " lanes)");
    for (const auto &l : body.bases) lines.push_back(l);
    lines.push_back("const int cl = w & " + str(L - 1) + ";");
    lines.push_back("double sum = 0.0;");
    const bool pairs = SplitLanesTakePairs(k);
    // eight loads in flight per lane (row sums of 1 024 terms: 69 % of the HBM peak with 4, 75 % with 8, 73 % with 16)
    lines.push_back(pairs ? "#pragma unroll 4" : "#pragma unroll 8");
    if (pairs)
        lines.push_back("for (int c = 2 * cl; c < " + str(s.contrCount) + "; c += " + str(2 * L) + ")");
    else
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
        if (pairs && has(r.idx, s.contr.back()))
        {
            // both terms of the pair in one load (through the ordinary pointer also for operands that scalar loads
            // would serve: the index differs from lane to lane here)
            const std::string at = src == kFromConstant ? PtrName(r.uvar) + "[" + ScalarBase(r) + Lit(uvars[r.uvar].viewOffset) + " + " + off + "]"
                                                        : PtrName(r.uvar) + "[o_k" + str(k) + "v" + str(v) + " + " + off + "]";
            lines.push_back("    const acro_pair p" + str(static_cast<long>(v)) + " = " +
                            (src == kFromGlobal && StreamedOnce(k, static_cast<int>(v)) ? "__builtin_nontemporal_load(reinterpret_cast<const acro_pair *>(&" + at + "));"
                                                                                         : "*reinterpret_cast<const acro_pair *>(&" + at + ");"));
            opnd = "p" + str(static_cast<long>(v)) + ".@";
        }
        else if (src == kFromConstant)
            opnd = ConstPtrName(r.uvar) + "[" + ScalarBase(r) + Lit(uvars[r.uvar].viewOffset) + " + " + off + "]";
        else if (lds)
            opnd = "lds[o_k" + str(k) + "v" + str(v) + " + " + off + "]";
        else
            opnd = GlobalRead(r.uvar, "o_k" + str(k) + "v" + str(v) + " + " + off, StreamedOnce(k, static_cast<int>(v)));
        prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
    }
    if (pairs)
    {
        for (const char *half : {"x", "y"})
        {
            std::string term = prod;
            for (size_t at = term.find('@'); at != std::string::npos; at = term.find('@')) term.replace(at, 1, half);
            lines.push_back("    sum += " + term + ";");
        }
    }
    else
    {
        lines.push_back("    sum += " + prod + ";");
    }
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

auto Generator::EmitLoopBody(int k, std::vector<std::string> &lines) -> void
{
    const Sub &s = subs[k];
    if (s.splitLanes > 0)
    {
        EmitSplitLanesBody(k, lines);
        return;
    }
    Body body;
    EmitBases(k, body);
    lines.push_back("// " + s.text + (s.tile.empty() ? "   (contraction as counted loops)" : "   (contraction as counted loops around a register tile)"));
    for (const auto &l : body.bases) lines.push_back(l);
    const long tc = s.tileCount;
    auto sumName = [&](long t) { return tc == 1 ? std::string("sum") : "sum_" + str(t); };
    for (long t = 0; t < tc; ++t) lines.push_back("double " + sumName(t) + " = 0.0;");
    // Which operands depend on the tile; the contraction indices that none of those carries go innermost, so that
    // what a tile entry reads is invariant in the inner loops and stays in (scalar) registers across them.
    std::vector<char> onTile(s.in.size(), 0);
    for (size_t v = 0; v < s.in.size(); ++v)
    {
        for (int id : s.in[v].idx) onTile[v] = onTile[v] || has(s.tile, id);
    }
    std::vector<int> order, inner;
    for (int c : s.contr)
    {
        bool carried = false;
        for (size_t v = 0; v < s.in.size(); ++v) carried = carried || (onTile[v] && has(s.in[v].idx, c));
        (carried || s.tile.empty() ? order : inner).push_back(c);
    }
    order.insert(order.end(), inner.begin(), inner.end());
    std::string indent;
    for (size_t j = 0; j < order.size(); ++j)
    {
        const std::string c = IdxVar(order[j]);
        // Around a register tile only the innermost loop is unrolled: with every loop unrolled the compiler requests
        // all scalar operands of all terms at once and spills them.
        if (j + 1 == order.size())
            lines.push_back(indent + (tc > 1 && extent[order[j]] <= 8 ? "#pragma unroll" : "#pragma unroll 4"));
        else if (tc > 1)
            lines.push_back(indent + "#pragma unroll 1");
        lines.push_back(indent + "for (int " + c + " = 0; " + c + " < " + str(extent[order[j]]) + "; ++" + c + ")");
        lines.push_back(indent + "{");
        indent += "    ";
    }
    std::vector<int> value(nidx, 0);
    auto operand = [&](size_t v) {
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
        const long fixed = LiteralOffset(r, s, lds, value);  // the tile entry's part (contraction values are zero)
        if (fixed != 0 || off.empty()) off += (off.empty() ? "" : " + ") + (lds ? str(fixed) : Lit(fixed));
        if (src == kFromConstant) return ConstPtrName(r.uvar) + "[" + ScalarBase(r) + Lit(uvars[r.uvar].viewOffset) + " + " + off + "]";
        if (lds) return "lds[o_k" + str(k) + "v" + str(v) + " + " + off + "]";
        return GlobalRead(r.uvar, "o_k" + str(k) + "v" + str(v) + " + " + off, StreamedOnce(k, static_cast<int>(v)));
    };
    std::string common;
    for (size_t v = 0; v < s.in.size(); ++v)
    {
        if (onTile[v]) continue;
        const std::string opnd = operand(v);
        common = common.empty() ? opnd : "(" + common + " * " + opnd + ")";
    }
    if (tc > 1 && !common.empty())
    {
        lines.push_back(indent + "const double common = " + common + ";");
        common = "common";
    }
    for (long t = 0; t < tc; ++t)
    {
        long rem = t;
        for (int j = static_cast<int>(s.tile.size()) - 1; j >= 0; --j)
        {
            value[s.tile[j]] = static_cast<int>(rem % extent[s.tile[j]]);
            rem /= extent[s.tile[j]];
        }
        std::string prod = common;
        for (size_t v = 0; v < s.in.size(); ++v)
        {
            if (!onTile[v]) continue;
            const std::string opnd = operand(v);
            prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
        }
        lines.push_back(indent + sumName(t) + " += " + prod + ";");
    }
    for (size_t j = 0; j < order.size(); ++j)
    {
        indent.resize(indent.size() - 4);
        lines.push_back(indent + "}");
    }
    for (long t = 0; t < tc; ++t)
    {
        long rem = t;
        for (int j = static_cast<int>(s.tile.size()) - 1; j >= 0; --j)
        {
            value[s.tile[j]] = static_cast<int>(rem % extent[s.tile[j]]);
            rem /= extent[s.tile[j]];
        }
        const long goff = LiteralOffset(s.out, s, false, value);
        const long loff = StoreOf(s.out.uvar).inLds ? LiteralOffset(s.out, s, true, value) : 0;
        const std::string gaddr = PtrName(s.out.uvar) + "[o_k" + str(k) + "g" + (tc > 1 ? " + " + Lit(goff) : std::string()) + "]";
        const std::string laddr = "lds[o_k" + str(k) + "l" + (tc > 1 ? " + " + str(loff) : std::string()) + "]";
        const std::string name = tc == 1 ? std::string("r") : "r_" + str(t);
        if (s.op == '=')
            lines.push_back("const double " + name + " = " + sumName(t) + ";");
        else
            lines.push_back("const double " + name + " = " + (OldValueInLds(k) ? laddr : gaddr) +
                            (s.op == '+' ? " + " : " - ") + sumName(t) + ";");
        if (NeedsLdsCopy(k)) lines.push_back(laddr + " = " + name + ";");
        if (StoresToGlobal(k) && !CopiesOutFromLds(k)) lines.push_back(GlobalStore(k, gaddr, name));
    }
}

}  // namespace codegen
}  // namespace acro
