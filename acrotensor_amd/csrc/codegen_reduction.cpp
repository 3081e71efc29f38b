// Kernel code generator, the reduction schedule (few outputs, long contraction) and the kernel-parameter helpers.
#include "hip_codegen_impl.hpp"
#include <limits>

namespace acro
{
namespace codegen
{

// Few outputs and a long contraction; or many outputs summed over a long contraction ("S_i_j = A_e_i_j" with 32 x 32
// outputs, "S_i = A_e_i B_e" with 5 000): as written such a kernel has one lane per output walk the whole contraction
// (0.2 - 6 % of the HBM peak).  With the outputs as the fastest dimension of the big operand any number of them is
// served (a lane per output, see EmitReduction), the other way round the finishing kernel holds up to 1 024.
auto Generator::ReductionServes(const Sub &s) const -> bool
{
    if (s.contrCount < kReductionMinContraction) return false;
    const long outputs = product(s.outIdx, extent);
    if (outputs <= envInt("ACRO_HIP_RED_MAX_OUTPUTS", kReductionMaxOutputs)) return true;
    if (envInt("ACRO_HIP_RED_WIDE") < 0 || s.in.empty()) return false;
    const VarRef *big = &s.in[0];
    for (const auto &r : s.in)
    {
        if (r.size > big->size) big = &r;
    }
    if (big->idx.empty()) return false;
    // a sum that streams the big operand, every value of which goes into one or two terms; a nest of contractions over
    // small operands ("Y_e_i = A_e_i_j_k B_j_l C_l_m D_m_i") is for the reordering to take apart instead
    if (static_cast<double>(outputs) * static_cast<double>(s.contrCount) > 2.0 * static_cast<double>(big->size)) return false;
    return has(s.outIdx, big->idx.back()) ? outputs <= 65536 : outputs <= 1024;
}

auto Generator::UseReductionSchedule() const -> bool
{
    if (subs.size() != 1 || NumGatherSlots() > 0) return false;
    const Sub &s = subs[0];
    if (s.out.repeated) return false;
    return ReductionServes(s);
}

// After the other schedules have declined and the generic plan is known: a kernel with a long contraction whose generic
// plan leaves each lane hundreds of terms and the device mostly idle (few outputs in any layout: "A_i_j += B_i_e C_j"
// with 12 x 16 outputs over 2^20 terms took 44 ms, "A_e += B_i C_e_i" with 2 048 rows of 8 192 terms 418 us for 134 MB)
// shares the contraction range out over workgroups instead.
auto Generator::UseReductionFallback() const -> bool
{
    if (subs.size() != 1 || factorised || NumGatherSlots() > 0 || envInt("ACRO_HIP_RED_FALLBACK") < 0) return false;
    const Sub &s = subs[0];
    if (s.out.repeated || s.matrixOp != 0 || s.in.empty() || s.contrCount < kReductionMinContraction) return false;
    bool anyDims = false;
    for (const auto &r : s.in) anyDims = anyDims || !r.idx.empty();
    const long outputs = product(s.outIdx, extent);
    if (!anyDims || outputs > 65536) return false;
    const long lanes = E * s.laneCount, each = s.contrCount / std::max(1, s.splitLanes);
    // (with more lanes than that the generic plan has the parallelism, and which of the two reads the smaller operands in
    // longer runs depends on their layout: "A_j_k += B_j_k_i C_j_i_e" with 57 344 outputs 3.0 ms as planned, 9.9 ms here)
    return each >= 256 && lanes <= 32768;
}

// Expression for the element offset of an occurrence given variables named i_<index> for every loop index.
auto Generator::FullOffset(const VarRef &r) const -> std::string
{
    std::string expr = uvars[r.uvar].viewOffset != 0 ? Lit(uvars[r.uvar].viewOffset) : std::string();
    for (size_t d = 0; d < r.idx.size(); ++d)
        expr += (expr.empty() ? "" : " + ") + IdxVar(r.idx[d]) + " * " + Lit(r.stride[d]);
    return expr.empty() ? "0" : expr;
}

// Kernel parameters: one pointer per storage, taken from a representative member occurrence.
// Storages that are kernel parameters: all but the intermediates of a factorised kernel, which are numbered last.
auto Generator::NumParamStores() const -> int
{
    int n = 0;
    for (const auto &st : stores)
    {
        if (!uvars[st.members[0]].isVirtual) ++n;
    }
    for (int si = 0; si < n; ++si) ACROBATIC_ASSERT(!uvars[stores[si].members[0]].isVirtual, "HIP generator: storage order");
    return n;
}

auto Generator::FillParams(HipKernelPlan &plan, bool honour_elision) const -> void
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

auto Generator::ParamList() const -> std::string
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

auto Generator::EmitReduction(HipKernelPlan &plan) -> void
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
    // Output entries and contraction terms are numbered in the memory order of the big operand (indices it does not
    // carry slowest), so that whichever of the two is laid along the lanes walks along its rows.  ("A_i_k = B_j_k_l C_e
    // D_k_j_e_i" numbered as written puts neighbouring lanes 16 MB apart in D: 2.9 ms for 170 MB.)
    auto inMemoryOrder = [&](std::vector<int> ids) {
        auto reach = [&](int id) {
            long st = 0;
            for (size_t d = 0; d < big->idx.size(); ++d)
            {
                if (big->idx[d] == id) st += big->stride[d];
            }
            return st == 0 ? std::numeric_limits<long>::max() : st;
        };
        std::stable_sort(ids.begin(), ids.end(), [&](int a, int b) { return reach(a) > reach(b); });
        return ids;
    };
    const std::vector<int> outIds = inMemoryOrder(s.outIdx), contrIds = inMemoryOrder(s.contr);
    // Few output entries that are the fastest dimension of the big operand ("S_i_j = A_n_i_j B_n"): a lane owns
    // whole contraction slices and keeps one accumulator per output entry ("pencil").  It reads the O entries of
    // its slice of A as 16-byte pieces and the slice's entry of B once, i.e. 6 load instructions per 80 bytes;
    // with one lane per (slice, output entry) every lane loads B again and the same bytes take 18 load
    // instructions (A alone streamed at 6.1 TB/s that way, A and B together at 5.0 - 5.5 TB/s).
    // The same for up to 64 outputs that are products of few loads ("A_i_j = B_e_i C_e_j" with 8 x 8 outputs: 16
    // loads and 64 accumulators per slice; one lane per (slice, output) reads every value eight times: 21.7 % of the
    // HBM peak).
    long loadsPerSlice = 0;
    for (const auto &r : s.in)
    {
        long n = 1;
        std::set<int> seen;
        for (int id : r.idx)
        {
            if (has(s.outIdx, id) && seen.insert(id).second) n *= extent[id];
        }
        loadsPerSlice += n;
    }
    const bool pencil = outputsFastest && (O <= 16 || (O <= 64 && 2 * loadsPerSlice <= O)) && envInt("ACRO_HIP_RED_PENCIL") >= 0;
    const int NTr = kReductionLanes;
    // The big operand streams through once, its values going into one term each, read by lanes that follow it through
    // memory in whole 128-byte lines per load instruction: requested with the non-temporal hint (64 column sums over 2^20
    // rows 75 -> 81 % of the HBM peak, 64 row sums 78 -> 84 %, 32 x 32 sums of element matrices 71 -> 74 %).  Not the
    // pencil form, whose lanes take 16-byte pieces of lines that their neighbours complete (2^20 slices of 3 x 3: 16.8 ->
    // 28.5 us), and not operands whose values go into several outputs (192 outputs by rows: 145 -> 238 us).
    const bool ntBig = envInt("ACRO_HIP_RED_NT") >= 0 && !pencil && !big->repeated && static_cast<double>(O) * static_cast<double>(Nc) <= static_cast<double>(big->size) &&
                       big->size % 16 == 0 && (outputsFastest ? O % 16 == 0 : big->ext.back() % 16 == 0);
    // Contraction index fastest and more than four outputs ("S_i = A_i_n" with 64 rows): with all outputs in every
    // workgroup only NTr / O lanes would walk along a row (32-byte pieces of 64 different rows per load
    // instruction).  Instead a workgroup takes four outputs, 64 adjacent lanes each, and the workgroups are dealt
    // out over groups of outputs as well as over the contraction range.
    const bool byRows = !pencil && !outputsFastest && O > 4 && NTr / O < 64 && (envInt("ACRO_HIP_ONE_PASS") <= 0 || O > NTr) &&
                        envInt("ACRO_HIP_RED_ROWS") >= 0;
    // More than 256 outputs that are the fastest dimension of the big operand ("S_i_j = A_e_i_j" with 16 x 16 outputs
    // and more): a workgroup takes 256 neighbouring outputs, a lane each, and a share of the contraction range; the
    // lanes of a wavefront read 512 consecutive bytes per term.  The finishing kernel has a workgroup per 256 outputs.
    const bool wide = !pencil && !byRows && O > NTr;   // (up to 256 outputs: a lane per output in every workgroup, below)
    // More outputs than one workgroup's lanes, whichever way they were summed: the finishing kernel has a workgroup per
    // 256 outputs too.
    const bool wideFinish = wide || O > 1024;
    const long Sn = pencil ? NTr : (byRows ? 64 : (wide ? 1 : NTr / O));  // contraction slices per workgroup and step
    // (Two neighbouring outputs per lane, read as one 16-byte piece, measured slower: "S_i_j = A_e_i_j" with 32 x 32
    // outputs over 131 072 entries 70 -> 60 % of the HBM peak.)
    const long Ow = NTr / Sn, Go = (byRows || wide) ? (O + Ow - 1) / Ow : 1;  // outputs per workgroup, groups of outputs
    // First-stage workgroups.  Pencil: one per CU (256 on this device) without unrolling, i.e. about 20 KB of
    // loads in flight per CU and one 4.7 MB window moving through the operands; more workgroups or deeper
    // unrolling measured slower at every n (n = 2^24: 206 us with 256 workgroups, 216 with 512, 252 with 2 048;
    // 214 / 263 us with the loop unrolled 2 / 4 times).  One lane per (slice, output entry): 8 bytes per lane
    // and load, so up to 512 workgroups and four loads in flight per lane (also swept: 256 - 8 192 workgroups,
    // unroll 1 - 8).
    const long G = (byRows || (wide && Go > 1)) ? std::min<long>(std::max<long>(1, 1024 / Go), std::max<long>(1, Nc / (Sn * 16)))
                                                : std::min<long>(pencil ? envInt("ACRO_HIP_RED_GROUPS", 256) : 512, std::max<long>(1, Nc / (Sn * (pencil ? 4 : 16))));
    // G counts the shares of the contraction range (rows of partials in the scratch buffer); the grid has one
    // workgroup per share and group of outputs.
    const long gridG = G * Go;
    // Lanes of the finishing kernel: enough for every lane to have all its loads of partials in flight at once
    // (the kernel is a chain of memory latencies: launch, one round of loads, LDS; 1024 lanes instead of 256
    // measured 16.8 instead of 17.2 us for the pair of launches at n = 2^20), at most 1024.  The one-pass
    // variant finishes with the lanes of the partial kernel.
    int NTf = NTr;
    const bool twoKernels = envInt("ACRO_HIP_ONE_PASS") <= 0 || wideFinish || O > NTr;
    if (twoKernels && !wideFinish)
    {
        NTf = kReductionLanes;
        while (NTf < 1024 && (G * O > NTf * 4 || NTf < O)) NTf *= 2;
    }
    const long S2 = wideFinish ? 1 : NTf / O;
    long wideParts = 1;   // lanes per output in the finishing kernel of the wide form
    while (wideFinish && wideParts < 16 && O * wideParts < 65536 && 8 * wideParts * 4 <= G) wideParts *= 4;

    const std::string dimName = mk.GetDimensionedNameString();
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx",
                  static_cast<unsigned long long>(hashString(dimName + "/reduction/" + (opt.noalias ? "n" : "a") +
                                                             (Positional() ? "p" : "u") +
                                                             (twoKernels ? "2" : (envInt("ACRO_HIP_ONE_PASS") >= 2 ? "1l" : "1")) + "/" + str(envInt("ACRO_HIP_RED_PENCIL")) +
                                                             (byRows ? "/rows" : (wide ? "/wide" : "")))));
    plan.module_name = std::string("acro_red_") + hex;
    const std::string fPartial = plan.module_name + "_partial", fFinal = plan.module_name + "_final";

    std::ostringstream sched;
    sched << "reduction schedule: " << O << " output entries, contraction of " << Nc << " terms split over " << G
          << " workgroups x " << Sn << " slices ("
          << (pencil ? "a lane owns whole slices"
                     : (byRows ? "four outputs per workgroup, 64 adjacent lanes along each"
                               : (wide ? "256 outputs per workgroup, a lane each"
                                       : (outputsFastest ? "output entries on adjacent lanes" : "slices on adjacent lanes"))))
          << "), partials added in a fixed order by "
          << (twoKernels ? "a second kernel" : "the workgroup that finishes last") << "\n  [0] " << s.text << "\n";
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
        out << "#pragma unroll " << envInt("ACRO_HIP_RED_UNROLL", 1) << "\n";
        out << "        for (long c = g * " << Sn << " + lane; c < " << Nc << "; c += " << G * Sn << ")\n        {\n";
        decompose(contrIds, "c", "            ");
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
            for (int j = static_cast<int>(outIds.size()) - 1; j >= 0; --j)
            {
                value[outIds[j]] = static_cast<int>(rem % extent[outIds[j]]);
                rem /= extent[outIds[j]];
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
                    const std::string at = PtrName(r.uvar) + "[ob" + str(static_cast<long>(v)) + " + " + Lit(lit) + "]";
                    loads.push_back("const double " + name + " = " + (ntBig && &r == big ? "__builtin_nontemporal_load(&" + at + ")" : at) + ";");
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
        decompose(outIds, "o", "        ");
        out << "#pragma unroll 4\n";   // (8: 77 -> 71 % of the HBM peak for 64 rows of 2^20 terms)
        out << "        for (long c = (long)gc * " << Sn << " + sl; c < " << Nc << "; c += " << G * Sn << ")\n        {\n";
        decompose(contrIds, "c", "            ");
        std::string prod;
        for (const auto &r : s.in)
        {
            const std::string opnd = (ntBig && &r == big) ? "__builtin_nontemporal_load(&" + PtrName(r.uvar) + "[" + FullOffset(r) + "])" : PtrName(r.uvar) + "[" + FullOffset(r) + "]";
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
    else if (wide)
    {
        out << "    const int og = blockIdx.x % " << Go << ", gc = blockIdx.x / " << Go << ";\n";
        out << "    const int o = og * " << Ow << " + lane;\n";
        out << "    if (o < " << O << ")\n    {\n";
        out << "        double sum = 0.0;\n";
        decompose(outIds, "o", "        ");
        out << "#pragma unroll 8\n";
        out << "        for (long c = gc; c < " << Nc << "; c += " << G << ")\n        {\n";
        decompose(contrIds, "c", "            ");
        std::string prod;
        for (const auto &r : s.in)
        {
            const std::string opnd = (ntBig && &r == big) ? "__builtin_nontemporal_load(&" + PtrName(r.uvar) + "[" + FullOffset(r) + "])" : PtrName(r.uvar) + "[" + FullOffset(r) + "]";
            prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
        }
        out << "            sum += " << prod << ";\n        }\n";
        out << "        scratch[(long)gc * " << O << " + o] = sum;\n    }\n}\n";
    }
    else
    {
        if (outputsFastest)
            out << "    const int sl = lane / " << O << ", o = lane % " << O << ";\n";
        else
            out << "    const int o = lane / " << Sn << ", sl = lane % " << Sn << ";\n";
        out << "    double sum = 0.0;\n";
        out << "    if (lane < " << Sn * O << ")\n    {\n";
        decompose(outIds, "o", "        ");
        out << "        const long g = " << gExpr << ";\n";
        out << "#pragma unroll 8\n";   // (4: 71 %, 8: 75 %, 16: 74 % of the HBM peak for 64 column sums over 2^20 rows)
        out << "        for (long c = g * " << Sn << " + sl; c < " << Nc << "; c += " << G * Sn << ")\n        {\n";
        decompose(contrIds, "c", "            ");
        std::string prod;
        for (const auto &r : s.in)
        {
            const std::string opnd = (ntBig && &r == big) ? "__builtin_nontemporal_load(&" + PtrName(r.uvar) + "[" + FullOffset(r) + "])" : PtrName(r.uvar) + "[" + FullOffset(r) + "]";
            prod = prod.empty() ? opnd : "(" + prod + " * " + opnd + ")";
        }
        out << "            sum += " << prod << ";\n        }\n    }\n";
        out << "    red[lane] = sum;\n    __syncthreads();\n";
        out << "    if (lane < " << O << ")\n    {\n        double t = 0.0;\n";
        out << "        for (int k = 0; k < " << Sn << "; ++k) t += red["
            << (outputsFastest ? "k * " + str(O) + " + lane" : "lane * " + str(Sn) + " + k") << "];\n";
    }
    if (byRows || wide)
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
        decompose(outIds, "lane", "        ");
        const std::string dst = (twoKernels ? std::string("result") : PtrName(s.out.uvar)) + "[" + FullOffset(s.out) + "]";
        if (s.op == '=')
            out << "        " << dst << " = t;\n";
        else
            out << "        " << dst << " = " << dst << (s.op == '+' ? " + t;\n" : " - t;\n");
        out << "    }\n";
    };
    if (wideFinish)
    {
        // a lane per output adds its partials in order; with few outputs and many shares, 4 or 16 lanes per output, each a
        // share of the partials, added through LDS in a fixed order again (1 024 outputs in 256 shares: 16.2 -> 4 us)
        out << "\nextern \"C\" __global__ __launch_bounds__(" << NTf << ") void " << fFinal << "(double *"
            << (opt.noalias ? "__restrict__ " : "") << "result, const double *__restrict__ scratch)\n{\n";
        const long each = NTf / wideParts;
        if (wideParts > 1)
        {
            out << "    __shared__ double red[" << NTf << "];\n";
            out << "    const int o = blockIdx.x * " << each << " + threadIdx.x % " << each << ", part = threadIdx.x / " << each << ";\n";
            out << "    double t = 0.0;\n";
            out << "    if (o < " << O << ")\n    {\n";
            out << "#pragma unroll 8\n";
            out << "        for (long g = part; g < " << G << "; g += " << wideParts << ") t += scratch[g * " << O << " + o];\n    }\n";
            out << "    red[threadIdx.x] = t;\n    __syncthreads();\n";
            out << "    if (part == 0 && o < " << O << ")\n    {\n";
            out << "#pragma unroll\n        for (int q = 1; q < " << wideParts << "; ++q) t += red[threadIdx.x + " << each << " * q];\n";
        }
        else
        {
            out << "    const int o = blockIdx.x * " << NTf << " + threadIdx.x;\n";
            out << "    if (o < " << O << ")\n    {\n        double t = 0.0;\n";
            out << "#pragma unroll 8\n";
            out << "        for (long g = 0; g < " << G << "; ++g) t += scratch[g * " << O << " + o];\n";
        }
        decompose(outIds, "o", "        ");
        const std::string dst = "result[" + FullOffset(s.out) + "]";
        if (s.op == '=')
            out << "        " << dst << " = t;\n";
        else
            out << "        " << dst << " = " << dst << (s.op == '+' ? " + t;\n" : " - t;\n");
        out << "    }\n}\n";
    }
    else if (twoKernels)
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
        fin.grid = wideFinish ? static_cast<unsigned>((O + NTf / wideParts - 1) / (NTf / wideParts)) : 1;
        fin.block = NTf;
        fin.params.push_back(uvars[s.out.uvar].storage);
        fin.params.push_back(-1);
        plan.launches.push_back(fin);
    }
}

}  // namespace codegen
}  // namespace acro
